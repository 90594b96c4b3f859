// Row permutes of the MoE layer (local scatter / gather) for gfx950.
//
// All of them move whole rows of `row_elems` elements between an expert-sorted
// buffer and a token/slot-ordered one, so they are bound by HBM bandwidth:
// a wave owns a 4 KiB piece of one row (64 lanes x 4 x 16-byte vectors), the
// row index is read once per wave, every lane issues its loads back to back
// before the first store, and the launch has one wave per piece so that all
// 256 CUs hold many independent requests.  Destination rows are written
// exactly once (zero rows included), so no separate zero-fill pass is needed
// and no floating-point atomics are used.
#include "permute.hpp"
#include "profile.hpp"

namespace fmoe {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kVecPerLane = 4;
constexpr int kPieceVecs = kWave * kVecPerLane;  // 256 x 16 B = 4 KiB

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ---- gather rows: out[r] = index[r] >= 0 ? inp[index[r]] : 0 -------------
// row_vecs = 16-byte vectors per row.
__global__ __launch_bounds__(kBlock) void gather_rows_vec_kernel(
    const u32x4 *__restrict__ inp, const int64_t *__restrict__ index, int64_t divisor,
    u32x4 *__restrict__ out, int64_t n_out, int64_t n_inp, int row_vecs, int pieces_per_row) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t piece = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t row = piece / pieces_per_row;
    if (row >= n_out) return;
    const int v0 = (int)(piece % pieces_per_row) * kPieceVecs;
    int64_t src = index[row];
    const bool live = src >= 0 && (src = src / divisor) < n_inp;
    u32x4 val[kVecPerLane];
#pragma unroll
    for (int j = 0; j < kVecPerLane; ++j) {
        const int v = v0 + j * kWave + lane;
        val[j] = u32x4{0, 0, 0, 0};
        if (live && v < row_vecs) val[j] = __builtin_nontemporal_load(&inp[src * row_vecs + v]);
    }
#pragma unroll
    for (int j = 0; j < kVecPerLane; ++j) {
        const int v = v0 + j * kWave + lane;
        if (v < row_vecs) __builtin_nontemporal_store(val[j], &out[row * row_vecs + v]);
    }
}

// element-wise fallback for rows that are not a whole number of aligned vectors
template <typename T>
__global__ __launch_bounds__(kBlock) void gather_rows_elem_kernel(
    const T *__restrict__ inp, const int64_t *__restrict__ index, int64_t divisor, T *__restrict__ out,
    int64_t n_out, int64_t n_inp, int64_t row_elems) {
    const int64_t row = blockIdx.x;
    int64_t src = index[row];
    const bool live = src >= 0 && (src = src / divisor) < n_inp;
    for (int64_t c = threadIdx.x; c < row_elems; c += kBlock)
        out[row * row_elems + c] = live ? inp[src * row_elems + c] : T(0);
}

// ---- scatter rows: out[index[r]] = inp[r] -----------------------------------
__global__ __launch_bounds__(kBlock) void scatter_rows_vec_kernel(
    const u32x4 *__restrict__ inp, const int64_t *__restrict__ index, u32x4 *__restrict__ out,
    int64_t n_in, int64_t n_out, int row_vecs, int pieces_per_row) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t piece = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t row = piece / pieces_per_row;
    if (row >= n_in) return;
    const int v0 = (int)(piece % pieces_per_row) * kPieceVecs;
    const int64_t dst = index[row];
    if (dst < 0 || dst >= n_out) return;
    u32x4 val[kVecPerLane];
#pragma unroll
    for (int j = 0; j < kVecPerLane; ++j) {
        const int v = v0 + j * kWave + lane;
        if (v < row_vecs) val[j] = __builtin_nontemporal_load(&inp[row * row_vecs + v]);
    }
#pragma unroll
    for (int j = 0; j < kVecPerLane; ++j) {
        const int v = v0 + j * kWave + lane;
        if (v < row_vecs) __builtin_nontemporal_store(val[j], &out[dst * row_vecs + v]);
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void scatter_rows_elem_kernel(
    const T *__restrict__ inp, const int64_t *__restrict__ index, T *__restrict__ out, int64_t n_in,
    int64_t n_out, int64_t row_elems) {
    const int64_t row = blockIdx.x;
    const int64_t dst = index[row];
    if (dst < 0 || dst >= n_out) return;
    for (int64_t c = threadIdx.x; c < row_elems; c += kBlock) out[dst * row_elems + c] = inp[row * row_elems + c];
}

// one wave per row; rows that are mapped are left alone
__global__ __launch_bounds__(kBlock) void zero_unmapped_kernel(
    const int64_t *__restrict__ index, unsigned char *__restrict__ out, int64_t n_out, int64_t row_bytes) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (row >= n_out || index[row] >= 0) return;
    unsigned char *dst = out + row * row_bytes;
    if ((row_bytes & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        for (int64_t b = lane * 16; b < row_bytes; b += kWave * 16) *(u32x4 *)(dst + b) = u32x4{0, 0, 0, 0};
    } else {
        for (int64_t b = lane; b < row_bytes; b += kWave) dst[b] = 0;
    }
}

// ---- inverse index --------------------------------------------------------
__global__ __launch_bounds__(kBlock) void fill_i64_kernel(int64_t *dst, int64_t n, int64_t value) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) dst[i] = value;
}

__global__ __launch_bounds__(kBlock) void invert_index_kernel(
    const int64_t *__restrict__ pos, int64_t n_pos, int64_t *__restrict__ inverse, int64_t n_out) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_pos) return;
    const int64_t p = pos[i];
    if (p >= 0 && p < n_out) inverse[p] = i;
}

// ---- fp32 accumulation over 16-byte vectors of T ---------------------------
template <typename T> struct VecOps;

template <> struct VecOps<float> {
    __device__ static void add(float (&acc)[8], const u32x4 &v) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += __uint_as_float(v[i]);
    }
    __device__ static u32x4 pack(const float (&acc)[8]) {
        return u32x4{__float_as_uint(acc[0]), __float_as_uint(acc[1]), __float_as_uint(acc[2]),
                     __float_as_uint(acc[3])};
    }
};

template <> struct VecOps<__bf16> {
    __device__ static void add(float (&acc)[8], const u32x4 &v) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] += __uint_as_float(v[i] << 16);
            acc[2 * i + 1] += __uint_as_float(v[i] & 0xffff0000u);
        }
    }
    __device__ static u32x4 pack(const float (&acc)[8]) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const __bf16 lo = (__bf16)acc[2 * i], hi = (__bf16)acc[2 * i + 1];
            r[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        return r;
    }
};

template <> struct VecOps<_Float16> {
    __device__ static void add(float (&acc)[8], const u32x4 &v) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] += (float)__builtin_bit_cast(_Float16, (uint16_t)(v[i] & 0xffffu));
            acc[2 * i + 1] += (float)__builtin_bit_cast(_Float16, (uint16_t)(v[i] >> 16));
        }
    }
    __device__ static u32x4 pack(const float (&acc)[8]) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const _Float16 lo = (_Float16)acc[2 * i], hi = (_Float16)acc[2 * i + 1];
            r[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        return r;
    }
};

// ---- reduce slots: out[t] = sum_j inp[slot_to_row[t*k+j]] ------------------
// A wave owns one 64-vector (1 KiB) piece of one output row, so the k source
// rows' loads are independent of each other.
constexpr int kMaxTopKRegs = 8;
template <typename T>
__global__ __launch_bounds__(kBlock) void reduce_slots_vec_kernel(
    const u32x4 *__restrict__ inp, const int64_t *__restrict__ slot_to_row, u32x4 *__restrict__ out,
    int64_t n_tokens, int top_k, int64_t n_inp, int row_vecs, int pieces_per_row) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t piece = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t t = piece / pieces_per_row;
    if (t >= n_tokens) return;
    const int v = (int)(piece % pieces_per_row) * kWave + lane;
    if (v >= row_vecs) return;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int j0 = 0; j0 < top_k; j0 += kMaxTopKRegs) {
        u32x4 val[kMaxTopKRegs];
        bool live[kMaxTopKRegs];
#pragma unroll
        for (int j = 0; j < kMaxTopKRegs; ++j) {
            live[j] = false;
            if (j0 + j < top_k) {
                const int64_t src = slot_to_row[t * top_k + j0 + j];
                live[j] = src >= 0 && src < n_inp;
                if (live[j]) val[j] = __builtin_nontemporal_load(&inp[src * row_vecs + v]);
            }
        }
#pragma unroll
        for (int j = 0; j < kMaxTopKRegs; ++j)
            if (live[j]) VecOps<T>::add(acc, val[j]);
    }
    __builtin_nontemporal_store(VecOps<T>::pack(acc), &out[t * row_vecs + v]);
}

template <typename T, typename Acc>
__global__ __launch_bounds__(kBlock) void reduce_slots_elem_kernel(
    const T *__restrict__ inp, const int64_t *__restrict__ slot_to_row, T *__restrict__ out,
    int64_t n_tokens, int top_k, int64_t n_inp, int64_t row_elems) {
    const int64_t t = blockIdx.x;
    for (int64_t c = threadIdx.x; c < row_elems; c += kBlock) {
        Acc acc = 0;
        for (int j = 0; j < top_k; ++j) {
            const int64_t src = slot_to_row[t * top_k + j];
            if (src >= 0 && src < n_inp) acc += (Acc)inp[src * row_elems + c];
        }
        out[t * row_elems + c] = (T)acc;
    }
}

// ---- general index_add: per-destination linked lists ------------------------
// head[r] / next[i] chain the source rows that land on destination r.  The
// chain order depends on scheduling, the SUM does not: the reducer always adds
// the sources of a row in ascending source index.
__global__ __launch_bounds__(kBlock) void link_rows_kernel(
    const int64_t *__restrict__ index, int64_t n_in, int64_t n_out,
    int32_t *__restrict__ head, int32_t *__restrict__ next) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_in) return;
    const int64_t r = index[i];
    if (r < 0 || r >= n_out) { next[i] = -1; return; }
    next[i] = atomicExch(&head[r], (int32_t)i);
}

__global__ __launch_bounds__(kBlock) void fill_i32_kernel(int32_t *dst, int64_t n, int32_t value) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) dst[i] = value;
}

constexpr int kSortSlots = 8;
// Walks the chain of destination row r and keeps the kSortSlots smallest source
// indices that are > after, ascending, INT32_MAX-padded.  Returns how many.
__device__ __forceinline__ int smallest_sources(const int32_t *__restrict__ next, int32_t first,
                                                int32_t after, int32_t (&slot)[kSortSlots]) {
#pragma unroll
    for (int s = 0; s < kSortSlots; ++s) slot[s] = INT32_MAX;
    int found = 0;
    for (int32_t i = first; i >= 0; i = next[i]) {
        if (i <= after) continue;
        ++found;
        int32_t x = i;
#pragma unroll
        for (int s = 0; s < kSortSlots; ++s) {
            const int32_t lo = x < slot[s] ? x : slot[s];
            const int32_t hi = x < slot[s] ? slot[s] : x;
            slot[s] = lo;
            x = hi;
        }
    }
    return found < kSortSlots ? found : kSortSlots;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void index_add_vec_kernel(
    const u32x4 *__restrict__ inp, const int32_t *__restrict__ head, const int32_t *__restrict__ next,
    u32x4 *__restrict__ out, int64_t n_out, int row_vecs, int pieces_per_row) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t piece = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t r = piece / pieces_per_row;
    if (r >= n_out) return;
    const int v = (int)(piece % pieces_per_row) * kWave + lane;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const int32_t first = head[r];
    int32_t after = -1;
    while (true) {
        int32_t slot[kSortSlots];
        const int n = smallest_sources(next, first, after, slot);
        if (n == 0) break;
        u32x4 val[kSortSlots];
#pragma unroll
        for (int s = 0; s < kSortSlots; ++s)
            if (s < n && v < row_vecs) val[s] = __builtin_nontemporal_load(&inp[(int64_t)slot[s] * row_vecs + v]);
#pragma unroll
        for (int s = 0; s < kSortSlots; ++s)
            if (s < n && v < row_vecs) VecOps<T>::add(acc, val[s]);
        if (n < kSortSlots) break;
        after = slot[kSortSlots - 1];
    }
    if (v < row_vecs) __builtin_nontemporal_store(VecOps<T>::pack(acc), &out[r * row_vecs + v]);
}

template <typename T, typename Acc>
__global__ __launch_bounds__(kBlock) void index_add_elem_kernel(
    const T *__restrict__ inp, const int32_t *__restrict__ head, const int32_t *__restrict__ next,
    T *__restrict__ out, int64_t n_out, int64_t row_elems) {
    const int64_t r = blockIdx.x;
    const int32_t first = head[r];
    for (int64_t c0 = 0; c0 < row_elems; c0 += kBlock) {
        const int64_t c = c0 + threadIdx.x;
        Acc acc = 0;
        int32_t after = -1;
        while (true) {
            int32_t slot[kSortSlots];
            const int n = smallest_sources(next, first, after, slot);
            if (n == 0) break;
            for (int s = 0; s < n; ++s)
                if (c < row_elems) acc += (Acc)inp[(int64_t)slot[s] * row_elems + c];
            if (n < kSortSlots) break;
            after = slot[kSortSlots - 1];
        }
        if (c < row_elems) out[r * row_elems + c] = (T)acc;
    }
}

bool vec_ok(const void *a, const void *b, int64_t row_elems, int dtype) {
    return aligned16(a) && aligned16(b) && (row_elems * dtype_bytes(dtype)) % 16 == 0;
}

int check_rows(const char *who, int64_t n_out, int64_t row_elems, int dtype) {
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "%s: unknown dtype %d", who, dtype);
    FMOE_REQUIRE(n_out >= 0 && row_elems >= 0, "%s: negative size", who);
    if (n_out > (int64_t)INT32_MAX || row_elems > (int64_t)(1 << 28))
        return fail(FMOE_ELIMIT, "%s: %lld rows x %lld elements is beyond the supported range", who,
                    (long long)n_out, (long long)row_elems);
    return FMOE_OK;
}

}  // namespace
}  // namespace fmoe

using namespace fmoe;

namespace fmoe {

int permute_gather_rows(const void *inp, const int64_t *index, int64_t divisor, void *out, int64_t n_out,
                        int64_t n_inp, int64_t row_elems, int dtype, hipStream_t st) {
    if (int rc = check_rows("gather_rows", n_out, row_elems, dtype)) return rc;
    FMOE_REQUIRE(divisor >= 1, "gather_rows: divisor=%lld", (long long)divisor);
    if (n_out == 0 || row_elems == 0) return FMOE_OK;
    FMOE_REQUIRE(index && out && (inp || n_inp == 0), "gather_rows: NULL pointer");
    ProfileScope prof(kProfGatherRows, 2.0 * n_out * row_elems * dtype_bytes(dtype), st);
    if (vec_ok(inp, out, row_elems, dtype)) {
        const int row_vecs = (int)(row_elems * dtype_bytes(dtype) / 16);
        const int ppr = (int)ceil_div(row_vecs, kPieceVecs);
        const int64_t blocks = ceil_div(n_out * ppr, kWavesPerBlock);
        if (blocks > INT32_MAX) return fail(FMOE_ELIMIT, "gather_rows: grid too large");
        gather_rows_vec_kernel<<<(int)blocks, kBlock, 0, st>>>((const u32x4 *)inp, index, divisor, (u32x4 *)out,
                                                                n_out, n_inp, row_vecs, ppr);
    } else {
        switch (dtype_bytes(dtype)) {
            case 2: gather_rows_elem_kernel<uint16_t><<<(int)n_out, kBlock, 0, st>>>((const uint16_t *)inp, index, divisor, (uint16_t *)out, n_out, n_inp, row_elems); break;
            case 4: gather_rows_elem_kernel<uint32_t><<<(int)n_out, kBlock, 0, st>>>((const uint32_t *)inp, index, divisor, (uint32_t *)out, n_out, n_inp, row_elems); break;
            default: gather_rows_elem_kernel<uint64_t><<<(int)n_out, kBlock, 0, st>>>((const uint64_t *)inp, index, divisor, (uint64_t *)out, n_out, n_inp, row_elems); break;
        }
    }
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

int permute_scatter_rows(const void *inp, const int64_t *index, void *out, int64_t n_in, int64_t n_out,
                         int64_t row_elems, int dtype, hipStream_t st) {
    if (int rc = check_rows("scatter_rows", n_in, row_elems, dtype)) return rc;
    if (n_in == 0 || row_elems == 0) return FMOE_OK;
    FMOE_REQUIRE(index && out && inp, "scatter_rows: NULL pointer");
    ProfileScope prof(kProfScatterRows, 2.0 * n_in * row_elems * dtype_bytes(dtype), st);
    if (vec_ok(inp, out, row_elems, dtype)) {
        const int row_vecs = (int)(row_elems * dtype_bytes(dtype) / 16);
        const int ppr = (int)ceil_div(row_vecs, kPieceVecs);
        const int64_t blocks = ceil_div(n_in * ppr, kWavesPerBlock);
        if (blocks > INT32_MAX) return fail(FMOE_ELIMIT, "scatter_rows: grid too large");
        scatter_rows_vec_kernel<<<(int)blocks, kBlock, 0, st>>>((const u32x4 *)inp, index, (u32x4 *)out, n_in, n_out,
                                                                 row_vecs, ppr);
    } else {
        switch (dtype_bytes(dtype)) {
            case 2: scatter_rows_elem_kernel<uint16_t><<<(int)n_in, kBlock, 0, st>>>((const uint16_t *)inp, index, (uint16_t *)out, n_in, n_out, row_elems); break;
            case 4: scatter_rows_elem_kernel<uint32_t><<<(int)n_in, kBlock, 0, st>>>((const uint32_t *)inp, index, (uint32_t *)out, n_in, n_out, row_elems); break;
            default: scatter_rows_elem_kernel<uint64_t><<<(int)n_in, kBlock, 0, st>>>((const uint64_t *)inp, index, (uint64_t *)out, n_in, n_out, row_elems); break;
        }
    }
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

int permute_zero_unmapped(const int64_t *index, void *out, int64_t n_out, int64_t row_elems, int dtype,
                          hipStream_t st) {
    if (int rc = check_rows("zero_unmapped", n_out, row_elems, dtype)) return rc;
    if (n_out == 0 || row_elems == 0) return FMOE_OK;
    FMOE_REQUIRE(index && out, "zero_unmapped: NULL pointer");
    zero_unmapped_kernel<<<(int)ceil_div(n_out, kWavesPerBlock), kBlock, 0, st>>>(
        index, (unsigned char *)out, n_out, row_elems * dtype_bytes(dtype));
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

namespace {

// ---- masked tokens: restore the full token order around the rows that went through the experts ----
// out[t,:] = row[t] >= 0 ? src[row[t],:] : (fill_row[t] >= 0 ? scale[t] * fill[fill_row[t],:] : 0)
// One workgroup per token row, threads stride over the row (coalesced).
template <typename T>
__global__ __launch_bounds__(kBlock) void mask_restore_kernel(
    const T *__restrict__ src, const int64_t *__restrict__ row, const T *__restrict__ scale,
    const T *__restrict__ fill, const int64_t *__restrict__ fill_row, T *__restrict__ out, int64_t n_src,
    int64_t n_fill, int64_t row_elems) {
    const int64_t t = blockIdx.x;
    const int64_t r = row[t];
    T *dst = out + t * row_elems;
    if (r >= 0 && r < n_src) {
        const T *s = src + r * row_elems;
        for (int64_t c = threadIdx.x; c < row_elems; c += kBlock) dst[c] = s[c];
        return;
    }
    const int64_t f = fill_row ? fill_row[t] : -1;
    if (f >= 0 && f < n_fill) {
        const float a = scale ? (float)scale[t] : 1.f;
        const T *s = fill + f * row_elems;
        for (int64_t c = threadIdx.x; c < row_elems; c += kBlock) dst[c] = (T)(a * (float)s[c]);
    } else {
        for (int64_t c = threadIdx.x; c < row_elems; c += kBlock) dst[c] = (T)0.f;
    }
}

// grad_scale[t] = masked token with a fill row ? <grad_out[t,:], fill[fill_row[t],:]> : 0, summed in a fixed
// order: every thread adds its strided share, the 256 partial sums are added in ascending order.
template <typename T>
__global__ __launch_bounds__(kBlock) void mask_scale_grad_kernel(
    const T *__restrict__ grad_out, const int64_t *__restrict__ row, const T *__restrict__ fill,
    const int64_t *__restrict__ fill_row, T *__restrict__ grad_scale, int64_t n_fill, int64_t row_elems) {
    __shared__ float part[kBlock];
    const int64_t t = blockIdx.x;
    const int64_t f = fill_row[t];
    float acc = 0.f;
    const bool masked = row[t] < 0 && f >= 0 && f < n_fill;
    if (masked) {
        const T *g = grad_out + t * row_elems, *s = fill + f * row_elems;
        for (int64_t c = threadIdx.x; c < row_elems; c += kBlock) acc += (float)g[c] * (float)s[c];
    }
    part[threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float sum = 0.f;
        if (masked)
            for (int i = 0; i < kBlock; ++i) sum += part[i];
        grad_scale[t] = (T)sum;
    }
}

}  // namespace
}  // namespace fmoe

extern "C" int fmoe_mask_restore(const void *src, const int64_t *token_to_row, const void *scale, const void *fill,
                                 const int64_t *fill_row, void *out, int64_t n_tokens, int64_t n_src, int64_t n_fill,
                                 int64_t row_elems, int dtype, void *stream) {
    FMOE_REQUIRE(n_tokens >= 0 && n_src >= 0 && n_fill >= 0 && row_elems >= 1, "fmoe_mask_restore: bad sizes");
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "fmoe_mask_restore: unknown dtype %d", dtype);
    if (n_tokens == 0) return FMOE_OK;
    if (n_tokens > (int64_t)INT32_MAX) return fail(FMOE_ELIMIT, "fmoe_mask_restore: %lld tokens", (long long)n_tokens);
    FMOE_REQUIRE(token_to_row && out && (src || n_src == 0) && ((fill && fill_row) || n_fill == 0),
                 "fmoe_mask_restore: NULL pointer");
    hipStream_t st = (hipStream_t)stream;
    const unsigned grid = (unsigned)n_tokens;
    switch (dtype) {
        case FMOE_F32: mask_restore_kernel<float><<<grid, kBlock, 0, st>>>((const float *)src, token_to_row, (const float *)scale, (const float *)fill, n_fill ? fill_row : nullptr, (float *)out, n_src, n_fill, row_elems); break;
        case FMOE_BF16: mask_restore_kernel<__bf16><<<grid, kBlock, 0, st>>>((const __bf16 *)src, token_to_row, (const __bf16 *)scale, (const __bf16 *)fill, n_fill ? fill_row : nullptr, (__bf16 *)out, n_src, n_fill, row_elems); break;
        case FMOE_F16: mask_restore_kernel<_Float16><<<grid, kBlock, 0, st>>>((const _Float16 *)src, token_to_row, (const _Float16 *)scale, (const _Float16 *)fill, n_fill ? fill_row : nullptr, (_Float16 *)out, n_src, n_fill, row_elems); break;
        default: mask_restore_kernel<double><<<grid, kBlock, 0, st>>>((const double *)src, token_to_row, (const double *)scale, (const double *)fill, n_fill ? fill_row : nullptr, (double *)out, n_src, n_fill, row_elems); break;
    }
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

extern "C" int fmoe_mask_scale_grad(const void *grad_out, const int64_t *token_to_row, const void *fill,
                                    const int64_t *fill_row, void *grad_scale, int64_t n_tokens, int64_t n_fill,
                                    int64_t row_elems, int dtype, void *stream) {
    FMOE_REQUIRE(n_tokens >= 0 && n_fill >= 1 && row_elems >= 1, "fmoe_mask_scale_grad: bad sizes");
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "fmoe_mask_scale_grad: unknown dtype %d", dtype);
    if (n_tokens == 0) return FMOE_OK;
    if (n_tokens > (int64_t)INT32_MAX) return fail(FMOE_ELIMIT, "fmoe_mask_scale_grad: %lld tokens", (long long)n_tokens);
    FMOE_REQUIRE(grad_out && token_to_row && fill && fill_row && grad_scale, "fmoe_mask_scale_grad: NULL pointer");
    hipStream_t st = (hipStream_t)stream;
    const unsigned grid = (unsigned)n_tokens;
    switch (dtype) {
        case FMOE_F32: mask_scale_grad_kernel<float><<<grid, kBlock, 0, st>>>((const float *)grad_out, token_to_row, (const float *)fill, fill_row, (float *)grad_scale, n_fill, row_elems); break;
        case FMOE_BF16: mask_scale_grad_kernel<__bf16><<<grid, kBlock, 0, st>>>((const __bf16 *)grad_out, token_to_row, (const __bf16 *)fill, fill_row, (__bf16 *)grad_scale, n_fill, row_elems); break;
        case FMOE_F16: mask_scale_grad_kernel<_Float16><<<grid, kBlock, 0, st>>>((const _Float16 *)grad_out, token_to_row, (const _Float16 *)fill, fill_row, (_Float16 *)grad_scale, n_fill, row_elems); break;
        default: return fail(FMOE_EINVAL, "fmoe_mask_scale_grad: float32, bfloat16 or float16 only");
    }
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

extern "C" int fmoe_gather_rows(const void *inp, const int64_t *index, void *out, int64_t n_out, int64_t n_inp,
                                int64_t row_elems, int dtype, void *stream) {
    return permute_gather_rows(inp, index, 1, out, n_out, n_inp, row_elems, dtype, (hipStream_t)stream);
}

extern "C" int fmoe_gather_rows_div(const void *inp, const int64_t *index, int64_t index_div, void *out,
                                    int64_t n_out, int64_t n_inp, int64_t row_elems, int dtype, void *stream) {
    return permute_gather_rows(inp, index, index_div, out, n_out, n_inp, row_elems, dtype, (hipStream_t)stream);
}

extern "C" int fmoe_invert_index(const int64_t *pos, int64_t n_pos, int64_t *inverse, int64_t n_out,
                                 void *stream) {
    FMOE_REQUIRE(n_pos >= 0 && n_out >= 0, "fmoe_invert_index: negative size");
    if (n_out == 0) return FMOE_OK;
    FMOE_REQUIRE(inverse && (pos || n_pos == 0), "fmoe_invert_index: NULL pointer");
    hipStream_t st = (hipStream_t)stream;
    fill_i64_kernel<<<(int)ceil_div(n_out, kBlock), kBlock, 0, st>>>(inverse, n_out, -1);
    FMOE_LAUNCH_CHECK();
    if (n_pos > 0) {
        invert_index_kernel<<<(int)ceil_div(n_pos, kBlock), kBlock, 0, st>>>(pos, n_pos, inverse, n_out);
        FMOE_LAUNCH_CHECK();
    }
    return FMOE_OK;
}

extern "C" int fmoe_reduce_slots(const void *inp, const int64_t *slot_to_row, void *out, int64_t n_tokens,
                                 int64_t top_k, int64_t n_inp, int64_t row_elems, int dtype, void *stream) {
    if (int rc = check_rows("fmoe_reduce_slots", n_tokens, row_elems, dtype)) return rc;
    FMOE_REQUIRE(top_k >= 1 && top_k <= 4096, "fmoe_reduce_slots: top_k=%lld", (long long)top_k);
    if (n_tokens == 0 || row_elems == 0) return FMOE_OK;
    FMOE_REQUIRE(slot_to_row && out && (inp || n_inp == 0), "fmoe_reduce_slots: NULL pointer");
    hipStream_t st = (hipStream_t)stream;
    // algorithmic bytes: every source row read once (n_inp), every token row written once
    ProfileScope prof(kProfReduceSlots, (double)(n_inp + n_tokens) * row_elems * dtype_bytes(dtype), st);
    const bool vec = vec_ok(inp, out, row_elems, dtype) && dtype != FMOE_F64;
    if (vec) {
        const int row_vecs = (int)(row_elems * dtype_bytes(dtype) / 16);
        const int ppr = (int)ceil_div(row_vecs, kWave);
        const int64_t blocks = ceil_div(n_tokens * ppr, kWavesPerBlock);
        if (blocks > INT32_MAX) return fail(FMOE_ELIMIT, "fmoe_reduce_slots: grid too large");
#define FMOE_RS(T) reduce_slots_vec_kernel<T><<<(int)blocks, kBlock, 0, st>>>((const u32x4 *)inp, slot_to_row, (u32x4 *)out, n_tokens, (int)top_k, n_inp, row_vecs, ppr)
        if (dtype == FMOE_F32) FMOE_RS(float);
        else if (dtype == FMOE_BF16) FMOE_RS(__bf16);
        else FMOE_RS(_Float16);
#undef FMOE_RS
    } else {
#define FMOE_RS(T, A) reduce_slots_elem_kernel<T, A><<<(int)n_tokens, kBlock, 0, st>>>((const T *)inp, slot_to_row, (T *)out, n_tokens, (int)top_k, n_inp, row_elems)
        if (dtype == FMOE_F32) FMOE_RS(float, float);
        else if (dtype == FMOE_BF16) FMOE_RS(__bf16, float);
        else if (dtype == FMOE_F16) FMOE_RS(_Float16, float);
        else FMOE_RS(double, double);
#undef FMOE_RS
    }
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

extern "C" int64_t fmoe_index_add_workspace_bytes(int64_t n_in, int64_t n_out) {
    if (n_in < 0 || n_out < 0) return 0;
    return (n_in + n_out) * (int64_t)sizeof(int32_t) + 64;
}

extern "C" int fmoe_index_add_rows(const void *inp, const int64_t *index, void *out, int64_t n_in, int64_t n_out,
                                   int64_t row_elems, int dtype, void *workspace, int64_t workspace_bytes,
                                   void *stream) {
    if (int rc = check_rows("fmoe_index_add_rows", n_out, row_elems, dtype)) return rc;
    FMOE_REQUIRE(n_in >= 0 && n_in <= (int64_t)INT32_MAX - 1, "fmoe_index_add_rows: n_in=%lld", (long long)n_in);
    if (n_out == 0 || row_elems == 0) return FMOE_OK;
    FMOE_REQUIRE(out && (n_in == 0 || (inp && index)), "fmoe_index_add_rows: NULL pointer");
    if (!workspace || workspace_bytes < fmoe_index_add_workspace_bytes(n_in, n_out))
        return fail(FMOE_EWORKSPACE, "fmoe_index_add_rows: workspace needs %lld bytes",
                    (long long)fmoe_index_add_workspace_bytes(n_in, n_out));
    hipStream_t st = (hipStream_t)stream;
    int32_t *head = (int32_t *)workspace;
    int32_t *next = head + n_out;
    fill_i32_kernel<<<(int)ceil_div(n_out, kBlock), kBlock, 0, st>>>(head, n_out, -1);
    FMOE_LAUNCH_CHECK();
    if (n_in > 0) {
        link_rows_kernel<<<(int)ceil_div(n_in, kBlock), kBlock, 0, st>>>(index, n_in, n_out, head, next);
        FMOE_LAUNCH_CHECK();
    }
    ProfileScope prof(kProfIndexAdd, (double)(n_in + n_out) * row_elems * dtype_bytes(dtype), st);
    const bool vec = vec_ok(inp, out, row_elems, dtype) && dtype != FMOE_F64;
    if (vec) {
        const int row_vecs = (int)(row_elems * dtype_bytes(dtype) / 16);
        const int ppr = (int)ceil_div(row_vecs, kWave);
        const int64_t blocks = ceil_div(n_out * ppr, kWavesPerBlock);
        if (blocks > INT32_MAX) return fail(FMOE_ELIMIT, "fmoe_index_add_rows: grid too large");
#define FMOE_IA(T) index_add_vec_kernel<T><<<(int)blocks, kBlock, 0, st>>>((const u32x4 *)inp, head, next, (u32x4 *)out, n_out, row_vecs, ppr)
        if (dtype == FMOE_F32) FMOE_IA(float);
        else if (dtype == FMOE_BF16) FMOE_IA(__bf16);
        else FMOE_IA(_Float16);
#undef FMOE_IA
    } else {
#define FMOE_IA(T, A) index_add_elem_kernel<T, A><<<(int)n_out, kBlock, 0, st>>>((const T *)inp, head, next, (T *)out, n_out, row_elems)
        if (dtype == FMOE_F32) FMOE_IA(float, float);
        else if (dtype == FMOE_BF16) FMOE_IA(__bf16, float);
        else if (dtype == FMOE_F16) FMOE_IA(_Float16, float);
        else FMOE_IA(double, double);
#undef FMOE_IA
    }
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}
