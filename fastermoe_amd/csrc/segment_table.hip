// Segment table in device memory (layout: grouped_gemm.hpp, namespace segtab).
//
// The grouped GEMMs need, per expert, the range of expert-sorted rows it owns, and per row tile
// the expert and rows it covers.  The host-count entry points build that table on the host from
// the CPU copy of the expert counts (as cuda/parallel_linear.cuh:69,85 walks expert_count on the
// host), which makes every layer call wait for a device-to-host read between the routing kernels
// and the first GEMM.  Here one small kernel builds the same table on the device, straight from
// the counts the routing kernels left there; the GEMMs launched over it are sized for the most
// tiles the rows can make and read the real numbers themselves.
#include "grouped_gemm.hpp"

namespace fmoe {
namespace {

constexpr int kTabBlock = 1024;

// One workgroup.  Pass 1: per expert (in chunks of kTabBlock, carrying the running sums) the
// exclusive prefixes of rows, 256-row tiles and 128-row tiles.  Counts are clamped so that their
// sum never exceeds rows_cap: the tile maps then never outgrow the space laid out for them,
// whatever the counts hold.  Pass 2: one thread per row tile finds its expert by binary search
// over the tile prefix and writes {expert, first row, rows, 0}.
__global__ __launch_bounds__(kTabBlock) void segment_table_kernel(const int64_t *__restrict__ counts, int n_expert,
                                                                  int rows_cap, int32_t *__restrict__ tab) {
    __shared__ int64_t row_sum[kTabBlock / kWave];
    __shared__ int32_t wave_sum[2][kTabBlock / kWave];
    __shared__ int32_t carry[3];  // rows (saturated at rows_cap), 256-row tiles, 128-row tiles so far
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    int32_t *seg = tab + segtab::seg_off();
    int32_t *pfx256 = tab + segtab::pfx256_off(n_expert);
    int32_t *pfx128 = tab + segtab::pfx128_off(n_expert);
    const int map256 = (int)segtab::map256_off(n_expert), map128 = (int)segtab::map128_off(rows_cap, n_expert);
    if (threadIdx.x < 3) carry[threadIdx.x] = 0;
    __syncthreads();
    for (int e0 = 0; e0 < n_expert; e0 += kTabBlock) {
        const int e = e0 + threadIdx.x;
        int64_t c64 = e < n_expert ? counts[e] : 0;
        c64 = c64 < 0 ? 0 : (c64 > rows_cap ? rows_cap : c64);
        // inclusive scans of (rows, tiles256, tiles128) over the workgroup; the row scan comes first
        // because the clamp of an expert's count depends on the rows before it
        // (int64: the sum of up to 1024 counts of up to rows_cap each)
        int64_t v = c64;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const int64_t up = __shfl_up(v, off, kWave);
            if (lane >= off) v += up;
        }
        if (lane == kWave - 1) row_sum[wave] = v;
        __syncthreads();
        int64_t before = carry[0];
        for (int w = 0; w < wave; ++w) before += row_sum[w];
        const int64_t incl = v + before;
        int64_t lo = incl - c64;
        lo = lo > rows_cap ? rows_cap : lo;
        const int64_t hi = incl > rows_cap ? rows_cap : incl;
        const int32_t rows = (int32_t)(hi - lo);  // this expert's rows after the clamp
        int32_t t[2] = {(rows + 255) / 256, (rows + 127) / 128};
        int32_t tv[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            int32_t s = t[k];
#pragma unroll
            for (int off = 1; off < kWave; off <<= 1) {
                const int32_t up = __shfl_up(s, off, kWave);
                if (lane >= off) s += up;
            }
            tv[k] = s;
            if (lane == kWave - 1) wave_sum[k][wave] = s;
        }
        __syncthreads();
        int32_t tb[2] = {carry[1], carry[2]};
        for (int w = 0; w < wave; ++w) { tb[0] += wave_sum[0][w]; tb[1] += wave_sum[1][w]; }
        if (e < n_expert) {
            seg[e] = (int32_t)lo;
            pfx256[e] = tb[0] + tv[0] - t[0];
            pfx128[e] = tb[1] + tv[1] - t[1];
        }
        __syncthreads();
        if (threadIdx.x == kTabBlock - 1) {
            // (the running row sum saturates at rows_cap, so it stays in int32 range)
            carry[0] = (int32_t)hi;
            carry[1] = tb[0] + tv[0];
            carry[2] = tb[1] + tv[1];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        seg[n_expert] = carry[0];
        pfx256[n_expert] = carry[1];
        pfx128[n_expert] = carry[2];
        tab[0] = n_expert;
        tab[segtab::kRows] = carry[0];
        tab[segtab::kTiles256] = carry[1];
        tab[segtab::kTiles128] = carry[2];
        tab[segtab::kMap256] = map256;
        tab[segtab::kMap128] = map128;
        tab[segtab::kRowsCap] = rows_cap;
        tab[7] = 0;
    }
    // the prefixes written above are read back below by other threads of this workgroup
    __threadfence();
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int block_rows = k == 0 ? 256 : 128;
        const int32_t *pfx = k == 0 ? pfx256 : pfx128;
        int32_t *map = tab + (k == 0 ? map256 : map128);
        const int tiles = carry[1 + k];
        for (int i = threadIdx.x; i < tiles; i += kTabBlock) {
            int lo = 0, hi = n_expert;  // pfx[lo] <= i < pfx[hi]
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (__builtin_nontemporal_load(pfx + mid) <= i) lo = mid; else hi = mid;
            }
            const int first = __builtin_nontemporal_load(seg + lo) + (i - __builtin_nontemporal_load(pfx + lo)) * block_rows;
            const int left = __builtin_nontemporal_load(seg + lo + 1) - first;
            int4 entry;
            entry.x = lo;
            entry.y = first;
            entry.z = left < block_rows ? left : block_rows;
            entry.w = 0;
            *(int4 *)(map + 4 * (int64_t)i) = entry;
        }
    }
}

}  // namespace
}  // namespace fmoe

using namespace fmoe;

extern "C" int64_t fmoe_segment_table_bytes(int64_t rows_cap, int64_t n_expert) {
    if (rows_cap < 0 || n_expert < 1) return 0;
    return segtab::total_ints(rows_cap, n_expert) * (int64_t)sizeof(int32_t);
}

extern "C" int fmoe_segment_table_build(const int64_t *expert_count, int64_t n_expert, int64_t rows_cap,
                                        void *segment_table, int64_t table_bytes, void *stream) {
    FMOE_REQUIRE(n_expert >= 1 && rows_cap >= 0, "fmoe_segment_table_build: n_expert=%lld rows_cap=%lld",
                 (long long)n_expert, (long long)rows_cap);
    if (n_expert > (int64_t)(1 << 24) || rows_cap > (int64_t)INT32_MAX - 65536)
        return fail(FMOE_ELIMIT, "fmoe_segment_table_build: %lld experts / %lld rows exceed the supported range",
                    (long long)n_expert, (long long)rows_cap);
    FMOE_REQUIRE(expert_count && segment_table, "fmoe_segment_table_build: NULL pointer");
    FMOE_REQUIRE((reinterpret_cast<uintptr_t>(segment_table) & 15u) == 0,
                 "fmoe_segment_table_build: the table must be 16-byte aligned");
    const int64_t need = fmoe_segment_table_bytes(rows_cap, n_expert);
    if (table_bytes < need)
        return fail(FMOE_EWORKSPACE, "fmoe_segment_table_build: the table needs %lld bytes, got %lld", (long long)need,
                    (long long)table_bytes);
    segment_table_kernel<<<1, kTabBlock, 0, (hipStream_t)stream>>>(expert_count, (int)n_expert, (int)rows_cap,
                                                                  (int32_t *)segment_table);
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}
