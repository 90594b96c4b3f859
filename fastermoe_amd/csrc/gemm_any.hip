// Grouped GEMM over ragged expert segments for what the 16-byte-chunk kernel does not take
// (gfx950): double precision -- the float64 rows of the reference's test grid,
// tests/test_numerical.py:84-94, cublasDgemm in cuda/utils/cublas_wrapper.h:46-93 -- on the fp64
// matrix pipe (v_mfma_f64_16x16x4_f64), and the 16- and 32-bit types with feature sizes or
// pointers off the 16-byte grid, converted to fp32 on the way into LDS and multiplied with
// v_mfma_f32_16x16x4_f32.
//
// A workgroup of four waves (2 x 2) computes a 64 x 64 tile of C, 32 x 32 per wave (2 x 2 MFMA
// blocks).  Slabs of 16 contraction elements go from memory through registers into LDS as
// [contraction][64 + 16 pad] doubles -- whichever way the operand lies in memory -- so that a
// fragment (one double per lane: row lane % 16 of the block, contraction element lane / 16 of the
// step) is a conflict-free 8-byte read; two stages, the next slab is fetched while the current one
// is multiplied.  Every element is bounds-checked on its own, so any feature size is taken.
// C's rows come from the A operand: lane l then holds, of a block, C(row l / 16 + 4 r, column l % 16)
// in double precision and C(row 4 (l / 16) + r, column l % 16) in single, r = 0..3, and 16 lanes
// store consecutive elements of a row.
#include "gemm_kernel.hpp"

namespace fmoe {
namespace {

typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kT = 64;        // tile edge
constexpr int kD = 16;        // contraction elements per slab
constexpr int kLd = kT + 16;  // LDS row length in doubles: k rows 640 bytes apart, half a bank cycle off
constexpr int kThreads64 = 256;

__device__ __forceinline__ double act_f64(double x, int act) {
    if (act == FMOE_ACT_RELU) return x > 0.0 ? x : 0.0;
    if (act == FMOE_ACT_GELU || act == gemm::kActGeluErf) return 0.5 * x * (1.0 + erf(x * 0.70710678118654752440));
    return x;
}
__device__ __forceinline__ double act_grad_f64(double x, int act) {
    if (act == FMOE_ACT_RELU) return x > 0.0 ? 1.0 : 0.0;
    if (act == FMOE_ACT_GELU || act == gemm::kActGeluErf)
        return 0.5 * (1.0 + erf(x * 0.70710678118654752440)) + x * 0.39894228040143267794 * exp(-0.5 * x * x);
    return 1.0;
}

__device__ __forceinline__ float act_of(float x, int act) { return gemm::apply_act<false>(x, act); }
__device__ __forceinline__ double act_of(double x, int act) { return act_f64(x, act); }
__device__ __forceinline__ float act_grad_of(float x, int act) { return gemm::act_grad<false>(x, act); }
__device__ __forceinline__ double act_grad_of(double x, int act) { return act_grad_f64(x, act); }

// T: element type in memory; A: type of the arithmetic (double for double, float for the rest).
// PSHAPE / QSHAPE as in the 16/32-bit kernel: kKC = [index][contraction] in memory, kMC = [contraction][index].
template <typename T, typename A, int PSHAPE, int QSHAPE, int RAGGED>
__global__ __launch_bounds__(kThreads64) void grouped_gemm_any_kernel(const gemm::GemmParams prm) {
    using namespace gemm;
    typedef typename std::conditional<sizeof(A) == 8, f64x4, f32x4>::type Acc;
    __shared__ A smem[2][2][kD][kLd];   // [stage][P, Q][contraction][index]
    const int ei = blockIdx.z;
    const int expert = prm.tab.first_expert + ei;
    const int seg_lo = prm.tab.seg[ei], seg_hi = prm.tab.seg[ei + 1];
    const int rows_total = RAGGED == kRaggedRows ? seg_hi - seg_lo : prm.n_rows;
    const int K = RAGGED == kRaggedRows ? prm.k_extent : seg_hi - seg_lo;
    const int n0 = blockIdx.x * kT;
    const int p_valid = min(kT, prm.n_cols - n0);
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wave_m0 = (wave >> 1) * 32, wave_n0 = (wave & 1) * 32;
    const int fi = lane & 15, fk = lane >> 4;
    const bool accumulate = RAGGED == kRaggedK && prm.accumulate_first && ei == 0;
    const T *bias = prm.bias ? (const T *)prm.bias + (int64_t)expert * prm.bias_expert_stride : nullptr;

    for (int m0 = blockIdx.y * kT; m0 < rows_total; m0 += gridDim.y * kT) {
        const int q_valid = min(kT, rows_total - m0);
        const T *Pb, *Qb;
        int64_t c_off;
        if (RAGGED == kRaggedRows) {
            const T *Pe = (const T *)prm.P + (int64_t)expert * prm.p_expert_stride;
            Pb = PSHAPE == kKC ? Pe + (int64_t)n0 * prm.ldp : Pe + n0;
            Qb = (const T *)prm.Q + (int64_t)(seg_lo + m0) * prm.ldq;
            c_off = (int64_t)(seg_lo + m0) * prm.ldc + n0;
        } else {
            Pb = (const T *)prm.P + (int64_t)seg_lo * prm.ldp + n0;
            Qb = (const T *)prm.Q + (int64_t)seg_lo * prm.ldq + m0;
            c_off = (int64_t)expert * prm.c_expert_stride + (int64_t)m0 * prm.ldc + n0;
        }
        // one operand's slab: 4 elements per thread, every one checked against the tile and the contraction
        A stage[2][4];
        auto fetch = [&](int which, int shape, const T *base, int64_t ld, int valid, int k0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int idx, k;
                if (shape == kKC) { idx = t >> 2; k = (t & 3) * 4 + j; }       // [idx][k]: 4 consecutive k of one idx
                else { k = t >> 4; idx = (t & 15) * 4 + j; }                   // [k][idx]: 4 consecutive idx of one k
                const bool ok = idx < valid && k0 + k < K;
                stage[which][j] = ok ? (A)(shape == kKC ? base[(int64_t)idx * ld + k0 + k] : base[(int64_t)(k0 + k) * ld + idx]) : (A)0;
            }
        };
        auto put = [&](int which, int shape, int buf) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int idx, k;
                if (shape == kKC) { idx = t >> 2; k = (t & 3) * 4 + j; }
                else { k = t >> 4; idx = (t & 15) * 4 + j; }
                smem[buf][which][k][idx] = stage[which][j];
            }
        };
        Acc acc[2][2];
#pragma unroll
        for (int by = 0; by < 2; ++by)
#pragma unroll
            for (int bx = 0; bx < 2; ++bx) acc[by][bx] = Acc{0, 0, 0, 0};
        const int n_slabs = (K + kD - 1) / kD;
        __syncthreads();   // the previous tile's reads of LDS are over
        if (n_slabs > 0) {
            fetch(0, PSHAPE, Pb, prm.ldp, p_valid, 0);
            fetch(1, QSHAPE, Qb, prm.ldq, q_valid, 0);
            put(0, PSHAPE, 0);
            put(1, QSHAPE, 0);
            __syncthreads();
        }
        for (int s = 0; s < n_slabs; ++s) {
            const int buf = s & 1;
            if (s + 1 < n_slabs) {
                fetch(0, PSHAPE, Pb, prm.ldp, p_valid, (s + 1) * kD);
                fetch(1, QSHAPE, Qb, prm.ldq, q_valid, (s + 1) * kD);
            }
#pragma unroll
            for (int ks = 0; ks < kD / 4; ++ks) {
                A a[2], b[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    a[i] = smem[buf][1][ks * 4 + fk][wave_m0 + 16 * i + fi];   // C's rows: the Q operand
                    b[i] = smem[buf][0][ks * 4 + fk][wave_n0 + 16 * i + fi];   // C's columns: the P operand
                }
#pragma unroll
                for (int by = 0; by < 2; ++by)
#pragma unroll
                    for (int bx = 0; bx < 2; ++bx) {
                        if constexpr (sizeof(A) == 8) acc[by][bx] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[by], b[bx], acc[by][bx], 0, 0, 0);
                        else acc[by][bx] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[by], b[bx], acc[by][bx], 0, 0, 0);
                    }
            }
            if (s + 1 < n_slabs) {
                put(0, PSHAPE, buf ^ 1);
                put(1, QSHAPE, buf ^ 1);
            }
            __syncthreads();
        }
        // epilogue: register r of a lane is row fk + 4 r (double) or 4 fk + r (single) of the block, column fi
        T *C = (T *)prm.C + c_off;
        const T *aux_in = prm.aux ? (const T *)prm.aux + c_off : nullptr;
        T *aux_out = prm.aux ? (T *)prm.aux + c_off : nullptr;
#pragma unroll
        for (int by = 0; by < 2; ++by)
#pragma unroll
            for (int bx = 0; bx < 2; ++bx)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = wave_m0 + 16 * by + (sizeof(A) == 8 ? fk + 4 * r : 4 * fk + r), col = wave_n0 + 16 * bx + fi;
                    if (row >= q_valid || col >= p_valid) continue;
                    const int64_t off = (int64_t)row * prm.ldc + col;
                    A v = acc[by][bx][r];
                    if (bias) v += (A)bias[n0 + col];
                    if (prm.epilogue == kEpiBiasAct) {
                        if (aux_out) aux_out[off] = (T)v;
                        v = act_of(v, prm.activation);
                    } else if (prm.epilogue == kEpiDAct) {
                        v *= act_grad_of((A)aux_in[off], prm.activation);
                    }
                    if (accumulate) v += (A)C[off];
                    C[off] = (T)v;
                }
    }
}

template <typename T, typename A>
int launch_any_typed(gemm::GemmParams &prm, int product, int epilogue, hipStream_t stream) {
    using namespace gemm;
    prm.epilogue = epilogue;
    const bool ragged_rows = product != 2;
    int max_rows = 0;
    if (ragged_rows) {
        for (int i = 0; i < prm.tab.n; ++i) max_rows = std::max(max_rows, prm.tab.seg[i + 1] - prm.tab.seg[i]);
    } else {
        max_rows = prm.n_rows;
    }
    if (max_rows == 0 || prm.n_cols == 0 || prm.tab.n == 0) return FMOE_OK;
    dim3 grid((unsigned)ceil_div(prm.n_cols, kT), (unsigned)std::min<int64_t>(ceil_div(max_rows, kT), 4096), (unsigned)prm.tab.n);
    ProfileScope prof(prm.profile_class, prm.profile_work, stream);
    switch (product) {
        case 0: grouped_gemm_any_kernel<T, A, kKC, kKC, kRaggedRows><<<grid, kThreads64, 0, stream>>>(prm); break;
        case 1: grouped_gemm_any_kernel<T, A, kMC, kKC, kRaggedRows><<<grid, kThreads64, 0, stream>>>(prm); break;
        default: grouped_gemm_any_kernel<T, A, kMC, kMC, kRaggedK><<<grid, kThreads64, 0, stream>>>(prm); break;
    }
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

}  // namespace

// product: 0 forward, 1 data gradient, 2 weight gradient.  Host-count segment tables only.
int launch_mfma_any(gemm::GemmParams &prm, int dtype, int product, int epilogue, hipStream_t stream) {
    switch (dtype) {
        case FMOE_F64: return launch_any_typed<double, double>(prm, product, epilogue, stream);
        case FMOE_F32: return launch_any_typed<float, float>(prm, product, epilogue, stream);
        case FMOE_BF16: return launch_any_typed<__bf16, float>(prm, product, epilogue, stream);
        case FMOE_F16: return launch_any_typed<_Float16, float>(prm, product, epilogue, stream);
    }
    return fail(FMOE_EINVAL, "unknown dtype %d", dtype);
}

}  // namespace fmoe
