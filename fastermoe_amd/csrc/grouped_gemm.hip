// Grouped GEMM over ragged expert segments for gfx950 (MI355X, CDNA4).
//
// One launch covers every expert: the row segments travel in the kernel
// arguments, a workgroup finds its (expert, row tile, column tile) by a binary
// search over the tile prefix, and there is no per-expert launch, no host loop
// over streams and no host synchronisation.
//
// Three products share one kernel template:
//   forward  Y[seg]  = X[seg] . W_e^T      rows ragged, contraction = in
//   dgrad    dX[seg] = dY[seg] . W_e       rows ragged, contraction = out
//   wgrad    dW_e    = dY[seg]^T . X[seg]  contraction ragged (the segment)
//
// This file holds the host side: segment tables, launch plans per product and per
// chunk and the stand-alone bias-gradient kernel that the any-shape kernel of gemm_any.hip (feature
// sizes that are not a multiple of 16 bytes, fp64) needs.  The MFMA
// kernel itself (tiling, LDS layouts, software pipeline, epilogues) is in
// gemm_kernel.hpp and is instantiated once per element type and product by
// gemm_inst.hip.
#include "gemm_kernel.hpp"
#include "profile.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <initializer_list>
#include <mutex>
#include <vector>

namespace fmoe {
using namespace gemm;
namespace {

// ---- bias gradient: column sums per expert segment ---------------------------------
// Thread (c, g) adds rows g, g+4, ... of column c in order; the four partial sums
// are then added in a fixed order, so the result is reproducible.
template <typename T, typename Acc>
__global__ __launch_bounds__(kThreads) void bias_grad_kernel(const T *__restrict__ gy, T *__restrict__ gb,
                                                             int64_t out_feat, const SegmentTable tab,
                                                             int accumulate_first) {
    __shared__ Acc part[4][64];
    const int ei = blockIdx.y;
    const int expert = tab.first_expert + ei;
    const int c = blockIdx.x * 64 + (threadIdx.x & 63);
    const int g = threadIdx.x >> 6;
    Acc acc = 0;
    if (c < out_feat)
        for (int r = tab.seg[ei] + g; r < tab.seg[ei + 1]; r += 4) acc += (Acc)gy[(int64_t)r * out_feat + c];
    part[g][threadIdx.x & 63] = acc;
    __syncthreads();
    if (g == 0 && c < out_feat) {
        Acc s = ((part[0][threadIdx.x] + part[1][threadIdx.x]) + part[2][threadIdx.x]) + part[3][threadIdx.x];
        T *dst = gb + (int64_t)expert * out_feat + c;
        if (accumulate_first && ei == 0) s += (Acc)*dst;
        *dst = (T)s;
    }
}

// ---- host side ---------------------------------------------------------------------------

struct Plan {
    int first, last;       // experts [first, last] covered (last < first: nothing)
    bool accumulate_first; // the first covered expert began before row_lo
};

// Row segments of experts [e0, e1] clipped to [row_lo, row_hi): seg[i] is the
// clipped start of expert e0+i, seg[n] the clipped end of expert e1.
void fill_table(SegmentTable *tab, const int64_t *counts, int e0, int e1, int64_t row_lo, int64_t row_hi,
                int block_rows) {
    auto clip = [&](int64_t r) { return r < row_lo ? row_lo : (r > row_hi ? row_hi : r); };
    int64_t start = 0;
    for (int e = 0; e < e0; ++e) start += counts[e];
    tab->n = e1 - e0 + 1;
    tab->first_expert = e0;
    int tiles = 0;
    for (int e = e0; e <= e1; ++e) {
        const int64_t end = start + counts[e];
        const int64_t lo = clip(start), hi = clip(end);
        tab->seg[e - e0] = (int32_t)lo;
        tab->seg[e - e0 + 1] = (int32_t)hi;
        tab->tile[e - e0] = tiles;
        tiles += (int)ceil_div(hi - lo, block_rows);
        start = end;
    }
    tab->tile[tab->n] = tiles;
}

// Tile of a launch.  256 x 256 (one workgroup per compute unit) unless that gives too few tiles
// to occupy the chip: then 128 x 256, and when even those number fewer than two per compute unit,
// 128 x 128 (two workgroups per compute unit).  (Lower tiles to cut the padding of short segments
// were measured and lost: with ~256 rows per expert the product is bound by streaming the weights,
// which a lower tile re-reads more often; and 128 x 128 tiles lose a quarter of the rate of large
// launches, because they read each operand from L2 and LDS more often per flop.)
// FMOE_GEMM_TILE=256x256|128x256|128x128 forces one shape (for tests and measurements).
struct TileShape {
    int bm, bn;
};
TileShape pick_tile(int64_t tiles_256) {
    if (const char *e = getenv("FMOE_GEMM_TILE")) {
        if (!strcmp(e, "256x256")) return {256, 256};
        if (!strcmp(e, "128x256")) return {128, 256};
        if (!strcmp(e, "128x128")) return {128, 128};
    }
    if (tiles_256 >= 512) return {256, 256};
    return tiles_256 >= 256 ? TileShape{128, 256} : TileShape{128, 128};
}

// The activation code the kernels see.  For results that are rounded to a 16-bit type GELU and its
// derivative come from polynomials (gemm_kernel.hpp); FMOE_GELU_ERF=1 selects the erf formula of
// the 32-bit path for them too (|error| <= 1.5e-7 instead of 4e-5 .. 1.4e-4, at about twice the
// epilogue's arithmetic).
int kernel_activation(int activation) {
    if (activation == FMOE_ACT_GELU) {
        const char *e = getenv("FMOE_GELU_ERF");
        if (e && e[0] == '1') return gemm::kActGeluErf;
    }
    return activation;
}

// ragged rows: tiles_256 counts every expert's rows rounded up to whole 256-row tiles
TileShape pick_rows_tile(const int64_t *counts, int64_t n_expert, int64_t row_lo, int64_t row_hi, int64_t n_cols) {
    int64_t start = 0, row_tiles = 0;
    for (int64_t e = 0; e < n_expert; ++e) {
        const int64_t end = start + counts[e];
        const int64_t lo = start < row_lo ? row_lo : start, hi = end > row_hi ? row_hi : end;
        if (hi > lo) row_tiles += ceil_div(hi - lo, 256);
        start = end;
    }
    return pick_tile(row_tiles * ceil_div(n_cols, 256));
}

// ragged rows over a device table: the host does not know the counts; rows_cap rows spread over
// the experts make about rows_cap / 256 whole tiles plus a partial one for every other expert
TileShape pick_rows_tile_estimate(int64_t rows_cap, int64_t n_expert, int64_t n_cols) {
    const int64_t whole = rows_cap / 256;
    return pick_tile((whole + std::min<int64_t>(n_expert, std::max<int64_t>(whole, 1)) / 2) * ceil_div(n_cols, 256));
}

// weight gradient: C is [out, in] per expert
TileShape pick_wgrad_tile(int64_t n_experts_written, int64_t out_feat, int64_t in_feat) {
    return pick_tile(n_experts_written * ceil_div(out_feat, 256) * ceil_div(in_feat, 256));
}

double table_flop(const SegmentTable &tab, int64_t in_feat, int64_t out_feat) {
    return 2.0 * (double)(tab.seg[tab.n] - tab.seg[0]) * (double)in_feat * (double)out_feat;
}

int check_counts(const char *who, const int64_t *counts, int64_t n_expert, int64_t row_lo, int64_t row_hi,
                 int64_t *total) {
    FMOE_REQUIRE(counts != nullptr, "%s: expert_count_host is NULL", who);
    FMOE_REQUIRE(n_expert >= 1, "%s: n_expert=%lld", who, (long long)n_expert);
    int64_t s = 0;
    for (int64_t e = 0; e < n_expert; ++e) {
        FMOE_REQUIRE(counts[e] >= 0, "%s: expert_count[%lld]=%lld is negative", who, (long long)e,
                     (long long)counts[e]);
        s += counts[e];
    }
    if (s > (int64_t)INT32_MAX || n_expert > (int64_t)(1 << 24))
        return fail(FMOE_ELIMIT, "%s: %lld rows / %lld experts exceed the supported range", who, (long long)s,
                    (long long)n_expert);
    FMOE_REQUIRE(row_lo >= 0 && row_lo <= row_hi && row_hi <= s, "%s: row range [%lld,%lld) outside [0,%lld]", who,
                 (long long)row_lo, (long long)row_hi, (long long)s);
    *total = s;
    return FMOE_OK;
}

// experts that own at least one row of [row_lo, row_hi)
Plan plan_rows(const int64_t *counts, int64_t n_expert, int64_t row_lo, int64_t row_hi) {
    Plan p{0, -1, false};
    int64_t start = 0;
    bool any = false;
    for (int e = 0; e < (int)n_expert; ++e) {
        const int64_t end = start + counts[e];
        if (end > row_lo && start < row_hi && end > start) {
            if (!any) { p.first = e; p.accumulate_first = start < row_lo; any = true; }
            p.last = e;
        }
        start = end;
    }
    return p;
}

// experts this chunk must WRITE in a ragged-K product: those with rows in the
// chunk, plus row-less experts positioned inside it.
Plan plan_contraction(const int64_t *counts, int64_t n_expert, int64_t row_lo, int64_t row_hi, bool last_chunk) {
    Plan p{0, -1, false};
    int64_t start = 0;
    bool any = false;
    for (int e = 0; e < (int)n_expert; ++e) {
        const int64_t end = start + counts[e];
        const bool has_rows = end > start && end > row_lo && start < row_hi;
        const bool empty_here = end == start && ((start >= row_lo && start < row_hi) || (last_chunk && start == row_hi));
        if (has_rows || empty_here) {
            if (!any) { p.first = e; p.accumulate_first = has_rows && start < row_lo; any = true; }
            p.last = e;
        }
        start = end;
    }
    return p;
}

template <typename T> bool fast_ok(std::initializer_list<const void *> ptrs, std::initializer_list<int64_t> dims) {
    constexpr int CE = 16 / (int)sizeof(T);
    for (const void *p : ptrs)
        if (p && !aligned16(p)) return false;
    // a row must be a whole number of 16-byte chunks, and 256 rows must stay inside the
    // 2 GiB a buffer offset can address
    for (int64_t d : dims)
        if (d % CE != 0 || d * (int64_t)sizeof(T) > (int64_t)(1 << 22)) return false;
    return true;
}

enum Product { kFwd = 0, kDgrad = 1, kWgrad = 2 };

struct SplitBuffer {
    int device;
    hipStream_t stream;
    float *ptr;
    size_t bytes;
};
std::mutex g_split_mutex;
std::vector<SplitBuffer> g_split_buffers;
int g_compute_units[16] = {};

template <int PRODUCT>
int dispatch(GemmParams &prm, int dtype, int epi, bool fast, hipStream_t stream) {
    // double precision, and shapes off the 16-byte grid: the element-checked kernel of gemm_any.hip
    if (!fast || dtype == FMOE_F64) return launch_mfma_any(prm, dtype, PRODUCT, epi, stream);
    switch (dtype * 3 + PRODUCT) {
        case FMOE_BF16 * 3 + kFwd: return launch_mfma_bf16_fwd(prm, epi, stream);
        case FMOE_BF16 * 3 + kDgrad: return launch_mfma_bf16_dgrad(prm, epi, stream);
        case FMOE_BF16 * 3 + kWgrad: return launch_mfma_bf16_wgrad(prm, epi, stream);
        case FMOE_F16 * 3 + kFwd: return launch_mfma_f16_fwd(prm, epi, stream);
        case FMOE_F16 * 3 + kDgrad: return launch_mfma_f16_dgrad(prm, epi, stream);
        case FMOE_F16 * 3 + kWgrad: return launch_mfma_f16_wgrad(prm, epi, stream);
        case FMOE_F32 * 3 + kFwd: return launch_mfma_f32_fwd(prm, epi, stream);
        case FMOE_F32 * 3 + kDgrad: return launch_mfma_f32_dgrad(prm, epi, stream);
        case FMOE_F32 * 3 + kWgrad: return launch_mfma_f32_wgrad(prm, epi, stream);
    }
    return fail(FMOE_EINVAL, "unknown dtype %d", dtype);
}

bool is_fast(int dtype, std::initializer_list<const void *> ptrs, std::initializer_list<int64_t> dims) {
    switch (dtype) {
        case FMOE_BF16: return fast_ok<__bf16>(ptrs, dims);
        case FMOE_F16: return fast_ok<_Float16>(ptrs, dims);
        case FMOE_F32: return fast_ok<float>(ptrs, dims);
    }
    return false;
}

}  // namespace

namespace gemm {

int device_compute_units() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return 256;
    std::lock_guard<std::mutex> lock(g_split_mutex);
    if (g_compute_units[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        g_compute_units[dev] = n;
    }
    return g_compute_units[dev];
}

// One buffer per (device, stream): launches on one stream run in order, so they can share it;
// launches on different streams may overlap and get their own.
float *split_workspace(hipStream_t stream, size_t bytes) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(g_split_mutex);
    for (SplitBuffer &b : g_split_buffers) {
        if (b.device != dev || b.stream != stream) continue;
        return b.bytes >= bytes ? b.ptr : nullptr;
    }
    if (g_split_buffers.size() >= 32) return nullptr;  // a process that keeps creating streams: stop splitting
    // a split launch never has more parts than compute units, each a tile of at most 256 x 256
    // floats: sized for that once, the buffer fits every later request
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    size_t want = (size_t)cus * 256 * 256 * sizeof(float);
    if (want < bytes) want = bytes;
    float *ptr = nullptr;
    if (hipMalloc((void **)&ptr, want) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    g_split_buffers.push_back(SplitBuffer{dev, stream, ptr, want});
    return ptr;
}

}  // namespace gemm

bool linear_forward_can_gather(const LinearForwardArgs &a) {
    if (a.dtype == FMOE_F64 || dtype_bytes(a.dtype) == 0) return false;
    if (!is_fast(a.dtype, {a.x, a.w, a.y, a.aux, a.bias}, {a.in_feat, a.out_feat})) return false;
    // (the loader divides 31-bit indices: every index that names a row must fit)
    if (a.x_index_div < 1 || a.x_index_div > (int64_t)INT32_MAX || a.x_total_rows < 0 ||
        a.x_total_rows > (int64_t)INT32_MAX / a.x_index_div)
        return false;
    return a.x_total_rows * a.in_feat * (int64_t)dtype_bytes(a.dtype) < ((int64_t)1 << 31);
}

// checks shared by the launches over a device table; fills the parts of prm that say so
int device_table_launch(const char *who, GemmParams &prm, const int32_t *dev_tab, int64_t rows_cap, int64_t n_expert,
                        bool fast) {
    FMOE_REQUIRE(fast, "%s: a launch over a device segment table needs 16-byte aligned tensors, feature sizes that are "
                       "multiples of 16 bytes and a 16- or 32-bit float type", who);
    FMOE_REQUIRE(n_expert >= 1 && n_expert <= (int64_t)(1 << 24) && rows_cap >= 0 && rows_cap <= (int64_t)INT32_MAX - 65536,
                 "%s: n_expert=%lld rows_cap=%lld", who, (long long)n_expert, (long long)rows_cap);
    FMOE_REQUIRE((reinterpret_cast<uintptr_t>(dev_tab) & 15u) == 0, "%s: the segment table must be 16-byte aligned", who);
    prm.dev_tab = dev_tab;
    prm.dev_rows_cap = rows_cap;
    prm.tab.n = (int32_t)n_expert;
    prm.tab.first_expert = 0;
    return FMOE_OK;
}

int64_t linear_dev_workspace_bytes(int64_t contraction, int dtype) {
    const int eb = dtype_bytes(dtype);
    if (eb == 0 || dtype == FMOE_F64 || contraction < 1) return 0;
    const int64_t per_slab = kSlabBytes / eb;
    if (!tail_split_possible((int)std::min<int64_t>(ceil_div(contraction, per_slab), 1 << 24), eb == 4 ? 2 : 1)) return 0;
    // one tile of fp32 accumulators per compute unit: a split never has more parts than that
    return (int64_t)device_compute_units() * 256 * 256 * (int64_t)sizeof(float);
}

int grouped_linear_forward(const LinearForwardArgs &a, const int64_t *counts, int64_t n_expert, int64_t row_lo,
                           int64_t row_hi, hipStream_t stream) {
    if (a.dev_tab != nullptr) {
        FMOE_REQUIRE(a.in_feat >= 1 && a.out_feat >= 1 && a.in_feat < (1 << 30) && a.out_feat < (1 << 30),
                     "linear_forward: in_feat=%lld out_feat=%lld", (long long)a.in_feat, (long long)a.out_feat);
        if (a.dev_rows_cap == 0) return FMOE_OK;
        FMOE_REQUIRE(a.x && a.w && a.y, "linear_forward: NULL tensor");
        const bool fast = is_fast(a.dtype, {a.x, a.w, a.y, a.aux, a.bias}, {a.in_feat, a.out_feat});
        FMOE_REQUIRE(a.x_row_index == nullptr || linear_forward_can_gather(a),
                     "linear_forward: rows cannot be gathered in the loader for this shape");
        const TileShape tile = pick_rows_tile_estimate(a.dev_rows_cap, n_expert, a.out_feat);
        GemmParams prm{};
        if (int rc = device_table_launch("linear_forward", prm, a.dev_tab, a.dev_rows_cap, n_expert, fast)) return rc;
        prm.block_m = tile.bm; prm.block_n = tile.bn;
        prm.profile_class = kProfGemmFwd; prm.profile_work = 2.0 * (double)a.dev_rows_cap * (double)a.in_feat * (double)a.out_feat;
        prm.P = a.w; prm.Q = a.x; prm.C = a.y; prm.bias = a.bias; prm.aux = a.aux;
        prm.q_row_index = a.x_row_index; set_row_index_divisor(prm, a.x_index_div); prm.q_total_rows = a.x_total_rows;
        prm.ldp = a.in_feat; prm.ldq = a.in_feat; prm.ldc = a.out_feat;
        prm.p_expert_stride = a.in_feat * a.out_feat;
        prm.bias_expert_stride = a.out_feat;
        prm.n_cols = (int)a.out_feat; prm.k_extent = (int)a.in_feat;
        prm.activation = kernel_activation(a.activation);
        const int64_t ws_need = linear_dev_workspace_bytes(a.in_feat, a.dtype);
        if (a.dev_workspace != nullptr && ws_need > 0 && a.dev_workspace_bytes >= ws_need && aligned16(a.dev_workspace))
            prm.dev_split_ws = (float *)a.dev_workspace;
        return dispatch<kFwd>(prm, a.dtype, a.epilogue, fast, stream);
    }
    int64_t total;
    if (int rc = check_counts("linear_forward", counts, n_expert, row_lo, row_hi, &total)) return rc;
    FMOE_REQUIRE(a.in_feat >= 1 && a.out_feat >= 1 && a.in_feat < (1 << 30) && a.out_feat < (1 << 30),
                 "linear_forward: in_feat=%lld out_feat=%lld", (long long)a.in_feat, (long long)a.out_feat);
    if (row_hi == row_lo) return FMOE_OK;
    FMOE_REQUIRE(a.x && a.w && a.y, "linear_forward: NULL tensor");
    const Plan plan = plan_rows(counts, n_expert, row_lo, row_hi);
    const bool fast = is_fast(a.dtype, {a.x, a.w, a.y, a.aux, a.bias}, {a.in_feat, a.out_feat});
    FMOE_REQUIRE(a.x_row_index == nullptr || linear_forward_can_gather(a),
                 "linear_forward: rows cannot be gathered in the loader for this shape");
    const TileShape tile = pick_rows_tile(counts, n_expert, row_lo, row_hi, a.out_feat);
    for (int e0 = plan.first; e0 <= plan.last; e0 += kMaxGroupExperts) {
        const int e1 = std::min(plan.last, e0 + kMaxGroupExperts - 1);
        GemmParams prm{};
        prm.block_m = tile.bm; prm.block_n = tile.bn;
        fill_table(&prm.tab, counts, e0, e1, row_lo, row_hi, tile.bm);
        prm.profile_class = kProfGemmFwd; prm.profile_work = table_flop(prm.tab, a.in_feat, a.out_feat);
        prm.P = a.w; prm.Q = a.x; prm.C = a.y; prm.bias = a.bias; prm.aux = a.aux;
        prm.q_row_index = a.x_row_index; set_row_index_divisor(prm, a.x_index_div); prm.q_total_rows = a.x_total_rows;
        prm.ldp = a.in_feat; prm.ldq = a.in_feat; prm.ldc = a.out_feat;
        prm.p_expert_stride = a.in_feat * a.out_feat;
        prm.bias_expert_stride = a.out_feat;
        prm.n_cols = (int)a.out_feat; prm.k_extent = (int)a.in_feat;
        prm.activation = kernel_activation(a.activation);
        if (int rc = dispatch<kFwd>(prm, a.dtype, a.epilogue, fast, stream)) return rc;
    }
    return FMOE_OK;
}

int grouped_linear_dgrad(const LinearDgradArgs &a, const int64_t *counts, int64_t n_expert, int64_t row_lo,
                         int64_t row_hi, hipStream_t stream) {
    if (a.dev_tab != nullptr) {
        FMOE_REQUIRE(a.in_feat >= 1 && a.out_feat >= 1 && a.in_feat < (1 << 30) && a.out_feat < (1 << 30),
                     "linear_dgrad: in_feat=%lld out_feat=%lld", (long long)a.in_feat, (long long)a.out_feat);
        if (a.dev_rows_cap == 0) return FMOE_OK;
        FMOE_REQUIRE(a.gy && a.w && a.gx, "linear_dgrad: NULL tensor");
        const bool fast = is_fast(a.dtype, {a.gy, a.w, a.gx, a.aux}, {a.in_feat, a.out_feat});
        const TileShape tile = pick_rows_tile_estimate(a.dev_rows_cap, n_expert, a.in_feat);
        GemmParams prm{};
        if (int rc = device_table_launch("linear_dgrad", prm, a.dev_tab, a.dev_rows_cap, n_expert, fast)) return rc;
        prm.block_m = tile.bm; prm.block_n = tile.bn;
        prm.profile_class = kProfGemmDgrad; prm.profile_work = 2.0 * (double)a.dev_rows_cap * (double)a.in_feat * (double)a.out_feat;
        prm.P = a.w; prm.Q = a.gy; prm.C = a.gx; prm.aux = const_cast<void *>(a.aux);
        prm.ldp = a.in_feat; prm.ldq = a.out_feat; prm.ldc = a.in_feat;
        prm.p_expert_stride = a.in_feat * a.out_feat;
        prm.n_cols = (int)a.in_feat; prm.k_extent = (int)a.out_feat;
        prm.activation = kernel_activation(a.activation);
        const int64_t ws_need = linear_dev_workspace_bytes(a.out_feat, a.dtype);
        if (a.dev_workspace != nullptr && ws_need > 0 && a.dev_workspace_bytes >= ws_need && aligned16(a.dev_workspace))
            prm.dev_split_ws = (float *)a.dev_workspace;
        return dispatch<kDgrad>(prm, a.dtype, a.epilogue, fast, stream);
    }
    int64_t total;
    if (int rc = check_counts("linear_dgrad", counts, n_expert, row_lo, row_hi, &total)) return rc;
    FMOE_REQUIRE(a.in_feat >= 1 && a.out_feat >= 1 && a.in_feat < (1 << 30) && a.out_feat < (1 << 30),
                 "linear_dgrad: in_feat=%lld out_feat=%lld", (long long)a.in_feat, (long long)a.out_feat);
    if (row_hi == row_lo) return FMOE_OK;
    FMOE_REQUIRE(a.gy && a.w && a.gx, "linear_dgrad: NULL tensor");
    const Plan plan = plan_rows(counts, n_expert, row_lo, row_hi);
    const bool fast = is_fast(a.dtype, {a.gy, a.w, a.gx, a.aux}, {a.in_feat, a.out_feat});
    const TileShape tile = pick_rows_tile(counts, n_expert, row_lo, row_hi, a.in_feat);
    for (int e0 = plan.first; e0 <= plan.last; e0 += kMaxGroupExperts) {
        const int e1 = std::min(plan.last, e0 + kMaxGroupExperts - 1);
        GemmParams prm{};
        prm.block_m = tile.bm; prm.block_n = tile.bn;
        fill_table(&prm.tab, counts, e0, e1, row_lo, row_hi, tile.bm);
        prm.profile_class = kProfGemmDgrad; prm.profile_work = table_flop(prm.tab, a.in_feat, a.out_feat);
        prm.P = a.w; prm.Q = a.gy; prm.C = a.gx; prm.aux = const_cast<void *>(a.aux);
        prm.ldp = a.in_feat; prm.ldq = a.out_feat; prm.ldc = a.in_feat;
        prm.p_expert_stride = a.in_feat * a.out_feat;
        prm.n_cols = (int)a.in_feat; prm.k_extent = (int)a.out_feat;
        prm.activation = kernel_activation(a.activation);
        if (int rc = dispatch<kDgrad>(prm, a.dtype, a.epilogue, fast, stream)) return rc;
    }
    return FMOE_OK;
}

int grouped_linear_wgrad(const LinearWgradArgs &a, const int64_t *counts, int64_t n_expert, int64_t row_lo,
                         int64_t row_hi, bool last_chunk, hipStream_t stream) {
    if (a.dev_tab != nullptr) {
        FMOE_REQUIRE(a.in_feat >= 1 && a.out_feat >= 1 && a.in_feat < (1 << 30) && a.out_feat < (1 << 30),
                     "linear_wgrad: in_feat=%lld out_feat=%lld", (long long)a.in_feat, (long long)a.out_feat);
        FMOE_REQUIRE(a.gw && (a.dev_rows_cap == 0 || (a.gy && a.x)), "linear_wgrad: NULL tensor");
        // (with no rows at all the pointers may be NULL: every expert's contraction is empty and nothing is read)
        const bool fast = is_fast(a.dtype, {a.gy, a.x, a.gw}, {a.in_feat, a.out_feat});
        const TileShape tile = pick_wgrad_tile(n_expert, a.out_feat, a.in_feat);
        GemmParams prm{};
        if (int rc = device_table_launch("linear_wgrad", prm, a.dev_tab, a.dev_rows_cap, n_expert, fast)) return rc;
        prm.block_m = tile.bm; prm.block_n = tile.bn;
        prm.profile_class = kProfGemmWgrad; prm.profile_work = 2.0 * (double)a.dev_rows_cap * (double)a.in_feat * (double)a.out_feat;
        prm.P = a.x; prm.Q = a.gy; prm.C = a.gw; prm.bias_grad = a.gb;
        prm.ldp = a.in_feat; prm.ldq = a.out_feat; prm.ldc = a.in_feat;
        prm.c_expert_stride = a.in_feat * a.out_feat;
        prm.n_cols = (int)a.in_feat; prm.n_rows = (int)a.out_feat;
        prm.accumulate_first = 0;
        return dispatch<kWgrad>(prm, a.dtype, kEpiStore, fast, stream);
    }
    int64_t total;
    if (int rc = check_counts("linear_wgrad", counts, n_expert, row_lo, row_hi, &total)) return rc;
    FMOE_REQUIRE(a.in_feat >= 1 && a.out_feat >= 1 && a.in_feat < (1 << 30) && a.out_feat < (1 << 30),
                 "linear_wgrad: in_feat=%lld out_feat=%lld", (long long)a.in_feat, (long long)a.out_feat);
    FMOE_REQUIRE(a.gw && (total == 0 || (a.gy && a.x)), "linear_wgrad: NULL tensor");
    const Plan plan = plan_contraction(counts, n_expert, row_lo, row_hi, last_chunk);
    const bool fast = is_fast(a.dtype, {a.gy, a.x, a.gw}, {a.in_feat, a.out_feat});
    const TileShape tile = pick_wgrad_tile(plan.last - plan.first + 1, a.out_feat, a.in_feat);
    for (int e0 = plan.first; e0 <= plan.last; e0 += kMaxGroupExperts) {
        const int e1 = std::min(plan.last, e0 + kMaxGroupExperts - 1);
        GemmParams prm{};
        prm.block_m = tile.bm; prm.block_n = tile.bn;
        fill_table(&prm.tab, counts, e0, e1, row_lo, row_hi, tile.bm);
        prm.profile_class = kProfGemmWgrad; prm.profile_work = table_flop(prm.tab, a.in_feat, a.out_feat);
        prm.P = a.x; prm.Q = a.gy; prm.C = a.gw; prm.bias_grad = fast ? a.gb : nullptr;
        prm.ldp = a.in_feat; prm.ldq = a.out_feat; prm.ldc = a.in_feat;
        prm.c_expert_stride = a.in_feat * a.out_feat;
        prm.n_cols = (int)a.in_feat; prm.n_rows = (int)a.out_feat;
        prm.accumulate_first = (e0 == plan.first && plan.accumulate_first) ? 1 : 0;
        if (int rc = dispatch<kWgrad>(prm, a.dtype, kEpiStore, fast, stream)) return rc;
    }
    // the MFMA kernel folds the bias gradient into its first column tiles; the any-shape path does not
    if (a.gb && !fast)
        return grouped_bias_grad(a.gy, a.gb, a.out_feat, a.dtype, counts, n_expert, row_lo, row_hi, last_chunk, stream);
    return FMOE_OK;
}

int grouped_bias_grad(const void *gy, void *gb, int64_t out_feat, int dtype, const int64_t *counts,
                      int64_t n_expert, int64_t row_lo, int64_t row_hi, bool last_chunk, hipStream_t stream) {
    int64_t total;
    if (int rc = check_counts("bias_grad", counts, n_expert, row_lo, row_hi, &total)) return rc;
    FMOE_REQUIRE(gb && (total == 0 || gy) && out_feat >= 1, "bias_grad: bad argument");
    const Plan plan = plan_contraction(counts, n_expert, row_lo, row_hi, last_chunk);
    for (int e0 = plan.first; e0 <= plan.last; e0 += kMaxGroupExperts) {
        const int e1 = std::min(plan.last, e0 + kMaxGroupExperts - 1);
        SegmentTable tab;
        fill_table(&tab, counts, e0, e1, row_lo, row_hi, 256);
        const int acc_first = (e0 == plan.first && plan.accumulate_first) ? 1 : 0;
        dim3 grid((unsigned)ceil_div(out_feat, 64), (unsigned)tab.n);
        ProfileScope prof(kProfBiasGrad, (double)(tab.seg[tab.n] - tab.seg[0]) * out_feat * dtype_bytes(dtype), stream);
        switch (dtype) {
            case FMOE_BF16: bias_grad_kernel<__bf16, float><<<grid, kThreads, 0, stream>>>((const __bf16 *)gy, (__bf16 *)gb, out_feat, tab, acc_first); break;
            case FMOE_F16: bias_grad_kernel<_Float16, float><<<grid, kThreads, 0, stream>>>((const _Float16 *)gy, (_Float16 *)gb, out_feat, tab, acc_first); break;
            case FMOE_F32: bias_grad_kernel<float, float><<<grid, kThreads, 0, stream>>>((const float *)gy, (float *)gb, out_feat, tab, acc_first); break;
            case FMOE_F64: bias_grad_kernel<double, double><<<grid, kThreads, 0, stream>>>((const double *)gy, (double *)gb, out_feat, tab, acc_first); break;
            default: return fail(FMOE_EINVAL, "bias_grad: unknown dtype %d", dtype);
        }
        FMOE_LAUNCH_CHECK();
    }
    return FMOE_OK;
}

}  // namespace fmoe

using namespace fmoe;

extern "C" int fmoe_gemm_tail_plan(int64_t total_tiles, int64_t contraction_slabs, int compute_units, int64_t *plan_host) {
    FMOE_REQUIRE(plan_host && total_tiles >= 0 && total_tiles < (int64_t)INT32_MAX && contraction_slabs >= 0 &&
                     contraction_slabs < (int64_t)INT32_MAX && compute_units >= 0,
                 "fmoe_gemm_tail_plan: bad argument");
    const gemm::TailSplit ts = gemm::plan_tail_split((int)total_tiles, (int)contraction_slabs,
                                                     compute_units > 0 ? compute_units : gemm::device_compute_units());
    plan_host[0] = ts.main_tiles;
    plan_host[1] = ts.k_split;
    plan_host[2] = ts.split_slabs;
    return FMOE_OK;
}

extern "C" int fmoe_linear_forward(const void *x, const void *w, const void *bias, void *y,
                                   const int64_t *expert_count_host, int64_t n_expert, int64_t in_feat,
                                   int64_t out_feat, int dtype, void *stream) {
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "fmoe_linear_forward: unknown dtype %d", dtype);
    int64_t total;
    if (int rc = check_counts("fmoe_linear_forward", expert_count_host, n_expert, 0, 0, &total)) return rc;
    LinearForwardArgs a{x, w, bias, y, nullptr, in_feat, out_feat, dtype, kEpiStore, FMOE_ACT_NONE};
    return grouped_linear_forward(a, expert_count_host, n_expert, 0, total, (hipStream_t)stream);
}

extern "C" int fmoe_linear_act_forward(const void *x, const void *w, const void *bias, void *pre, void *y,
                                       const int64_t *expert_count_host, int64_t n_expert, int64_t in_feat,
                                       int64_t out_feat, int dtype, int activation, void *stream) {
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "fmoe_linear_act_forward: unknown dtype %d", dtype);
    FMOE_REQUIRE(activation >= FMOE_ACT_NONE && activation <= FMOE_ACT_GELU, "fmoe_linear_act_forward: activation %d",
                 activation);
    int64_t total;
    if (int rc = check_counts("fmoe_linear_act_forward", expert_count_host, n_expert, 0, 0, &total)) return rc;
    LinearForwardArgs a{x, w, bias, y, pre, in_feat, out_feat, dtype, kEpiBiasAct, activation};
    return grouped_linear_forward(a, expert_count_host, n_expert, 0, total, (hipStream_t)stream);
}

extern "C" int fmoe_linear_dact_backward(const void *grad_y, const void *w, const void *pre, void *grad_x,
                                         const int64_t *expert_count_host, int64_t n_expert, int64_t in_feat,
                                         int64_t out_feat, int dtype, int activation, void *stream) {
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "fmoe_linear_dact_backward: unknown dtype %d", dtype);
    FMOE_REQUIRE(activation >= FMOE_ACT_NONE && activation <= FMOE_ACT_GELU,
                 "fmoe_linear_dact_backward: activation %d", activation);
    int64_t total;
    if (int rc = check_counts("fmoe_linear_dact_backward", expert_count_host, n_expert, 0, 0, &total)) return rc;
    FMOE_REQUIRE(activation == FMOE_ACT_NONE || total == 0 || pre != nullptr, "fmoe_linear_dact_backward: pre is NULL");
    const bool has_act = activation != FMOE_ACT_NONE;
    LinearDgradArgs d{grad_y, w, grad_x, has_act ? pre : nullptr, in_feat, out_feat, dtype,
                      has_act ? kEpiDAct : kEpiStore, activation};
    return grouped_linear_dgrad(d, expert_count_host, n_expert, 0, total, (hipStream_t)stream);
}

extern "C" int fmoe_linear_backward(const void *grad_y, const void *x, const void *w, void *grad_x, void *grad_w,
                                    void *grad_b, const int64_t *expert_count_host, int64_t n_expert,
                                    int64_t in_feat, int64_t out_feat, int dtype, void *stream) {
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "fmoe_linear_backward: unknown dtype %d", dtype);
    int64_t total;
    if (int rc = check_counts("fmoe_linear_backward", expert_count_host, n_expert, 0, 0, &total)) return rc;
    hipStream_t st = (hipStream_t)stream;
    if (grad_x) {
        LinearDgradArgs d{grad_y, w, grad_x, nullptr, in_feat, out_feat, dtype, kEpiStore, FMOE_ACT_NONE};
        if (int rc = grouped_linear_dgrad(d, expert_count_host, n_expert, 0, total, st)) return rc;
    }
    if (grad_w) {
        LinearWgradArgs g{grad_y, x, grad_w, grad_b, in_feat, out_feat, dtype};
        if (int rc = grouped_linear_wgrad(g, expert_count_host, n_expert, 0, total, true, st)) return rc;
    } else if (grad_b) {
        if (int rc = grouped_bias_grad(grad_y, grad_b, out_feat, dtype, expert_count_host, n_expert, 0, total, true, st))
            return rc;
    }
    return FMOE_OK;
}

// ---- the same products over a segment table in device memory ---------------------------------

extern "C" int fmoe_linear_dev_supported(int64_t in_feat, int64_t out_feat, int dtype) {
    const int eb = dtype_bytes(dtype);
    if (eb == 0 || dtype == FMOE_F64 || in_feat < 1 || out_feat < 1) return 0;
    const int64_t ce = 16 / eb;
    return (in_feat % ce == 0 && out_feat % ce == 0 && in_feat * eb <= (1 << 22) && out_feat * eb <= (1 << 22)) ? 1 : 0;
}

extern "C" int64_t fmoe_linear_dev_workspace_bytes(int64_t contraction, int dtype) {
    return linear_dev_workspace_bytes(contraction, dtype);
}

extern "C" int fmoe_linear_forward_dev(const void *x, const int64_t *x_row_index, int64_t x_index_div,
                                       int64_t x_total_rows, const void *w, const void *bias, void *pre, void *y,
                                       const void *segment_table, int64_t n_expert, int64_t rows_cap, int64_t in_feat,
                                       int64_t out_feat, int dtype, int activation, void *workspace,
                                       int64_t workspace_bytes, void *stream) {
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "fmoe_linear_forward_dev: unknown dtype %d", dtype);
    FMOE_REQUIRE(activation >= FMOE_ACT_NONE && activation <= FMOE_ACT_GELU, "fmoe_linear_forward_dev: activation %d",
                 activation);
    FMOE_REQUIRE(segment_table != nullptr, "fmoe_linear_forward_dev: NULL segment table");
    FMOE_REQUIRE(x_row_index == nullptr || (x_index_div >= 1 && x_total_rows >= 0),
                 "fmoe_linear_forward_dev: x_index_div=%lld x_total_rows=%lld", (long long)x_index_div, (long long)x_total_rows);
    const bool plain = activation == FMOE_ACT_NONE && pre == nullptr;
    LinearForwardArgs a{x, w, bias, y, pre, in_feat, out_feat, dtype, plain ? kEpiStore : kEpiBiasAct, activation};
    a.x_row_index = x_row_index;
    a.x_index_div = x_row_index ? x_index_div : 1;
    a.x_total_rows = x_row_index ? x_total_rows : 0;
    a.dev_tab = (const int32_t *)segment_table;
    a.dev_rows_cap = rows_cap;
    a.dev_workspace = workspace;
    a.dev_workspace_bytes = workspace_bytes;
    return grouped_linear_forward(a, nullptr, n_expert, 0, rows_cap, (hipStream_t)stream);
}

extern "C" int fmoe_linear_dgrad_dev(const void *grad_y, const void *w, const void *pre, void *grad_x,
                                     const void *segment_table, int64_t n_expert, int64_t rows_cap, int64_t in_feat,
                                     int64_t out_feat, int dtype, int activation, void *workspace,
                                     int64_t workspace_bytes, void *stream) {
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "fmoe_linear_dgrad_dev: unknown dtype %d", dtype);
    FMOE_REQUIRE(activation >= FMOE_ACT_NONE && activation <= FMOE_ACT_GELU, "fmoe_linear_dgrad_dev: activation %d",
                 activation);
    FMOE_REQUIRE(segment_table != nullptr, "fmoe_linear_dgrad_dev: NULL segment table");
    FMOE_REQUIRE(activation == FMOE_ACT_NONE || rows_cap == 0 || pre != nullptr, "fmoe_linear_dgrad_dev: pre is NULL");
    const bool has_act = activation != FMOE_ACT_NONE;
    LinearDgradArgs d{grad_y, w, grad_x, has_act ? pre : nullptr, in_feat, out_feat, dtype,
                      has_act ? kEpiDAct : kEpiStore, activation};
    d.dev_tab = (const int32_t *)segment_table;
    d.dev_rows_cap = rows_cap;
    d.dev_workspace = workspace;
    d.dev_workspace_bytes = workspace_bytes;
    return grouped_linear_dgrad(d, nullptr, n_expert, 0, rows_cap, (hipStream_t)stream);
}

extern "C" int fmoe_linear_wgrad_dev(const void *grad_y, const void *x, void *grad_w, void *grad_b,
                                     const void *segment_table, int64_t n_expert, int64_t rows_cap, int64_t in_feat,
                                     int64_t out_feat, int dtype, void *stream) {
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "fmoe_linear_wgrad_dev: unknown dtype %d", dtype);
    FMOE_REQUIRE(segment_table != nullptr, "fmoe_linear_wgrad_dev: NULL segment table");
    LinearWgradArgs g{grad_y, x, grad_w, grad_b, in_feat, out_feat, dtype};
    g.dev_tab = (const int32_t *)segment_table;
    g.dev_rows_cap = rows_cap;
    return grouped_linear_wgrad(g, nullptr, n_expert, 0, rows_cap, true, (hipStream_t)stream);
}
