// Score-weighted combination of a token's top-k expert outputs (gfx950):
//   out[t,:] = sum_j score[t,j] * x[t*k + j,:]
// i.e. the bmm of [N,1,k] x [N,k,d] that ends the MoE layer, and its backward.
// With a row index (`idx`, the slot -> expert-sorted row map) the same kernels read
// the experts' output rows where they lie, x[idx[t*k + j],:], so the copy back to
// slot order and the combine become one pass; a negative index is a dropped slot.
// These are k tiny dot products per token: as a batched GEMM they are bound by
// launch geometry, as a streaming kernel they are bound by HBM bandwidth, which
// is what this file does -- 16-byte loads, fp32 accumulation, one rounding.
#include "common.hpp"
#include "profile.hpp"

namespace fmoe {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Vec;  // 16 bytes of T <-> floats
template <> struct Vec<float> {
    static constexpr int N = 4;
    __device__ static void unpack(const u32x4 &v, float (&f)[8]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(v[i]);
    }
    __device__ static u32x4 pack(const float (&f)[8]) {
        return u32x4{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
    }
};
template <> struct Vec<__bf16> {
    static constexpr int N = 8;
    __device__ static void unpack(const u32x4 &v, float (&f)[8]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(v[i] << 16);
            f[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
        }
    }
    __device__ static u32x4 pack(const float (&f)[8]) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const __bf16 lo = (__bf16)f[2 * i], hi = (__bf16)f[2 * i + 1];
            r[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        return r;
    }
};
template <> struct Vec<_Float16> {
    static constexpr int N = 8;
    __device__ static void unpack(const u32x4 &v, float (&f)[8]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v[i] & 0xffffu));
            f[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v[i] >> 16));
        }
    }
    __device__ static u32x4 pack(const float (&f)[8]) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const _Float16 lo = (_Float16)f[2 * i], hi = (_Float16)f[2 * i + 1];
            r[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        return r;
    }
};

// row of x that slot s reads or writes: s itself, or idx[s] (negative or beyond n_rows: none)
__device__ __forceinline__ int64_t slot_row(const int64_t *idx, int64_t s, int64_t n_rows) {
    if (idx == nullptr) return s;
    const int64_t r = idx[s];
    return (r >= 0 && r < n_rows) ? r : -1;
}

// forward, vector path: a wave owns 64 vectors (1 KiB) of one output row
template <typename T>
__global__ __launch_bounds__(kBlock) void combine_fwd_vec_kernel(
    const u32x4 *__restrict__ x, const int64_t *__restrict__ idx, int64_t n_rows, const T *__restrict__ score,
    u32x4 *__restrict__ out, int64_t n_tokens, int top_k, int row_vecs, int pieces_per_row) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t piece = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t t = piece / pieces_per_row;
    if (t >= n_tokens) return;
    const int v = (int)(piece % pieces_per_row) * kWave + lane;
    if (v >= row_vecs) return;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int j0 = 0; j0 < top_k; j0 += 8) {
        u32x4 val[8];
        float w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (j0 + j < top_k) {
                const int64_t r = slot_row(idx, t * top_k + j0 + j, n_rows);
                w[j] = r >= 0 ? (float)score[t * top_k + j0 + j] : 0.f;
                val[j] = r >= 0 ? __builtin_nontemporal_load(&x[r * row_vecs + v]) : u32x4{0, 0, 0, 0};
            }
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (j0 + j < top_k) {
                float f[8];
                Vec<T>::unpack(val[j], f);
#pragma unroll
                for (int i = 0; i < Vec<T>::N; ++i) acc[i] += w[j] * f[i];
            }
    }
    __builtin_nontemporal_store(Vec<T>::pack(acc), &out[t * row_vecs + v]);
}

template <typename T, typename Acc>
__global__ __launch_bounds__(kBlock) void combine_fwd_elem_kernel(
    const T *__restrict__ x, const int64_t *__restrict__ idx, int64_t n_rows, const T *__restrict__ score,
    T *__restrict__ out, int64_t n_tokens, int top_k, int64_t row_elems) {
    const int64_t t = blockIdx.x;
    for (int64_t c = threadIdx.x; c < row_elems; c += kBlock) {
        Acc acc = 0;
        for (int j = 0; j < top_k; ++j) {
            const int64_t r = slot_row(idx, t * top_k + j, n_rows);
            if (r >= 0) acc += (Acc)score[t * top_k + j] * (Acc)x[r * row_elems + c];
        }
        out[t * row_elems + c] = (T)acc;
    }
}

// backward: one workgroup per token.  grad_x[t*k+j,:] = score[t,j] * grad_out[t,:];
// grad_score[t,j] = <grad_out[t,:], x[t*k+j,:]>, reduced lane -> wave -> workgroup in a
// fixed order.
template <typename Acc>
__device__ __forceinline__ Acc block_sum(Acc v, Acc *scratch) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_down(v, off, kWave);
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[wave] = v;
    __syncthreads();
    Acc s = 0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) s += scratch[w];
    return s;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void combine_bwd_vec_kernel(
    const u32x4 *__restrict__ grad_out, const u32x4 *__restrict__ x, const int64_t *__restrict__ idx, int64_t n_rows,
    const T *__restrict__ score, u32x4 *__restrict__ grad_x, T *__restrict__ grad_score, int top_k, int row_vecs) {
    __shared__ float scratch[kWavesPerBlock];
    const int64_t t = blockIdx.x;
    for (int j = 0; j < top_k; ++j) {
        const float w = (float)score[t * top_k + j];
        const int64_t row = slot_row(idx, t * top_k + j, n_rows);  // uniform over the workgroup
        float dot = 0.f;
        if (row >= 0) {
            for (int v = threadIdx.x; v < row_vecs; v += kBlock) {
                float g[8], f[8], r[8];
                Vec<T>::unpack(grad_out[t * row_vecs + v], g);
                Vec<T>::unpack(__builtin_nontemporal_load(&x[row * row_vecs + v]), f);
#pragma unroll
                for (int i = 0; i < Vec<T>::N; ++i) {
                    dot += g[i] * f[i];
                    r[i] = w * g[i];
                }
                __builtin_nontemporal_store(Vec<T>::pack(r), &grad_x[row * row_vecs + v]);
            }
        }
        const float total = block_sum<float>(dot, scratch);
        if (threadIdx.x == 0) grad_score[t * top_k + j] = (T)total;
    }
}

template <typename T, typename Acc>
__global__ __launch_bounds__(kBlock) void combine_bwd_elem_kernel(
    const T *__restrict__ grad_out, const T *__restrict__ x, const int64_t *__restrict__ idx, int64_t n_rows,
    const T *__restrict__ score, T *__restrict__ grad_x, T *__restrict__ grad_score, int top_k, int64_t row_elems) {
    __shared__ Acc scratch[kWavesPerBlock];
    const int64_t t = blockIdx.x;
    for (int j = 0; j < top_k; ++j) {
        const Acc w = (Acc)score[t * top_k + j];
        const int64_t row = slot_row(idx, t * top_k + j, n_rows);
        Acc dot = 0;
        if (row >= 0) {
            for (int64_t c = threadIdx.x; c < row_elems; c += kBlock) {
                const Acc g = (Acc)grad_out[t * row_elems + c];
                dot += g * (Acc)x[row * row_elems + c];
                grad_x[row * row_elems + c] = (T)(w * g);
            }
        }
        const Acc total = block_sum<Acc>(dot, scratch);
        if (threadIdx.x == 0) grad_score[t * top_k + j] = (T)total;
    }
}

int check(const char *who, int64_t n_tokens, int64_t top_k, int64_t row_elems, int dtype) {
    FMOE_REQUIRE(dtype_bytes(dtype) != 0, "%s: unknown dtype %d", who, dtype);
    FMOE_REQUIRE(n_tokens >= 0 && top_k >= 1 && row_elems >= 0, "%s: bad sizes", who);
    if (n_tokens > (int64_t)INT32_MAX || top_k > 65536 || row_elems > (int64_t)(1 << 28))
        return fail(FMOE_ELIMIT, "%s: sizes beyond the supported range", who);
    return FMOE_OK;
}

bool vec_ok(std::initializer_list<const void *> ptrs, int64_t row_elems, int dtype) {
    if (dtype == FMOE_F64 || (row_elems * dtype_bytes(dtype)) % 16 != 0) return false;
    for (const void *p : ptrs)
        if (!aligned16(p)) return false;
    return true;
}

}  // namespace
}  // namespace fmoe

using namespace fmoe;

namespace {

int combine_forward_impl(const char *who, const void *x, const int64_t *idx, int64_t n_rows, const void *score, void *out,
                         int64_t n_tokens, int64_t top_k, int64_t row_elems, int dtype, void *stream) {
    if (int rc = check(who, n_tokens, top_k, row_elems, dtype)) return rc;
    if (n_tokens == 0 || row_elems == 0) return FMOE_OK;
    FMOE_REQUIRE(score && out && (x || n_rows == 0), "%s: NULL pointer", who);
    hipStream_t st = (hipStream_t)stream;
    ProfileScope prof(kProfCombine, (double)(top_k + 1) * n_tokens * row_elems * dtype_bytes(dtype), st);
    if (vec_ok({x, out}, row_elems, dtype)) {
        const int row_vecs = (int)(row_elems * dtype_bytes(dtype) / 16);
        const int ppr = (int)ceil_div(row_vecs, kWave);
        const int64_t blocks = ceil_div(n_tokens * ppr, kWavesPerBlock);
        if (blocks > INT32_MAX) return fail(FMOE_ELIMIT, "%s: grid too large", who);
#define FMOE_CF(T) combine_fwd_vec_kernel<T><<<(int)blocks, kBlock, 0, st>>>((const u32x4 *)x, idx, n_rows, (const T *)score, (u32x4 *)out, n_tokens, (int)top_k, row_vecs, ppr)
        if (dtype == FMOE_F32) FMOE_CF(float);
        else if (dtype == FMOE_BF16) FMOE_CF(__bf16);
        else FMOE_CF(_Float16);
#undef FMOE_CF
    } else {
#define FMOE_CF(T, A) combine_fwd_elem_kernel<T, A><<<(int)n_tokens, kBlock, 0, st>>>((const T *)x, idx, n_rows, (const T *)score, (T *)out, n_tokens, (int)top_k, row_elems)
        if (dtype == FMOE_F32) FMOE_CF(float, float);
        else if (dtype == FMOE_BF16) FMOE_CF(__bf16, float);
        else if (dtype == FMOE_F16) FMOE_CF(_Float16, float);
        else FMOE_CF(double, double);
#undef FMOE_CF
    }
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

int combine_backward_impl(const char *who, const void *grad_out, const void *x, const int64_t *idx, int64_t n_rows,
                          const void *score, void *grad_x, void *grad_score, int64_t n_tokens, int64_t top_k,
                          int64_t row_elems, int dtype, void *stream) {
    if (int rc = check(who, n_tokens, top_k, row_elems, dtype)) return rc;
    if (n_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE(grad_out && score && grad_score && ((x && grad_x) || n_rows == 0), "%s: NULL pointer", who);
    hipStream_t st = (hipStream_t)stream;
    ProfileScope prof(kProfCombine, (double)(2 * top_k + 1) * n_tokens * row_elems * dtype_bytes(dtype), st);
    if (vec_ok({grad_out, x, grad_x}, row_elems, dtype)) {
        const int row_vecs = (int)(row_elems * dtype_bytes(dtype) / 16);
#define FMOE_CB(T) combine_bwd_vec_kernel<T><<<(int)n_tokens, kBlock, 0, st>>>((const u32x4 *)grad_out, (const u32x4 *)x, idx, n_rows, (const T *)score, (u32x4 *)grad_x, (T *)grad_score, (int)top_k, row_vecs)
        if (dtype == FMOE_F32) FMOE_CB(float);
        else if (dtype == FMOE_BF16) FMOE_CB(__bf16);
        else FMOE_CB(_Float16);
#undef FMOE_CB
    } else {
#define FMOE_CB(T, A) combine_bwd_elem_kernel<T, A><<<(int)n_tokens, kBlock, 0, st>>>((const T *)grad_out, (const T *)x, idx, n_rows, (const T *)score, (T *)grad_x, (T *)grad_score, (int)top_k, row_elems)
        if (dtype == FMOE_F32) FMOE_CB(float, float);
        else if (dtype == FMOE_BF16) FMOE_CB(__bf16, float);
        else if (dtype == FMOE_F16) FMOE_CB(_Float16, float);
        else FMOE_CB(double, double);
#undef FMOE_CB
    }
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

}  // namespace

extern "C" int fmoe_combine_forward(const void *x, const void *score, void *out, int64_t n_tokens, int64_t top_k,
                                    int64_t row_elems, int dtype, void *stream) {
    return combine_forward_impl("fmoe_combine_forward", x, nullptr, n_tokens * top_k, score, out, n_tokens, top_k,
                                row_elems, dtype, stream);
}

extern "C" int fmoe_combine_backward(const void *grad_out, const void *x, const void *score, void *grad_x,
                                     void *grad_score, int64_t n_tokens, int64_t top_k, int64_t row_elems,
                                     int dtype, void *stream) {
    return combine_backward_impl("fmoe_combine_backward", grad_out, x, nullptr, n_tokens * top_k, score, grad_x,
                                 grad_score, n_tokens, top_k, row_elems, dtype, stream);
}

extern "C" int fmoe_gather_combine_forward(const void *rows, const int64_t *slot_to_row, const void *score, void *out,
                                           int64_t n_tokens, int64_t top_k, int64_t n_rows, int64_t row_elems,
                                           int dtype, void *stream) {
    FMOE_REQUIRE(slot_to_row != nullptr || n_tokens == 0, "fmoe_gather_combine_forward: slot_to_row is NULL");
    FMOE_REQUIRE(n_rows >= 0 && n_rows <= n_tokens * top_k, "fmoe_gather_combine_forward: n_rows=%lld", (long long)n_rows);
    return combine_forward_impl("fmoe_gather_combine_forward", rows, slot_to_row, n_rows, score, out, n_tokens, top_k,
                                row_elems, dtype, stream);
}

extern "C" int fmoe_gather_combine_backward(const void *grad_out, const void *rows, const int64_t *slot_to_row,
                                            const void *score, void *grad_rows, void *grad_score, int64_t n_tokens,
                                            int64_t top_k, int64_t n_rows, int64_t row_elems, int dtype,
                                            void *stream) {
    FMOE_REQUIRE(slot_to_row != nullptr || n_tokens == 0, "fmoe_gather_combine_backward: slot_to_row is NULL");
    FMOE_REQUIRE(n_rows >= 0 && n_rows <= n_tokens * top_k, "fmoe_gather_combine_backward: n_rows=%lld", (long long)n_rows);
    return combine_backward_impl("fmoe_gather_combine_backward", grad_out, rows, slot_to_row, n_rows, score, grad_rows,
                                 grad_score, n_tokens, top_k, row_elems, dtype, stream);
}
