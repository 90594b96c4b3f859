// Device side of the grouped GEMM: kernel template and its launcher.  Included by
// gemm_inst.hip (one translation unit per element type and product, so that the
// variants build in parallel) and by grouped_gemm.hip (host dispatch).
#pragma once
#include "grouped_gemm.hpp"
#include "profile.hpp"

#include <algorithm>
#include <atomic>
#include <mutex>
#include <type_traits>

namespace fmoe {
namespace gemm {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Waves of a workgroup along C's rows and columns.  Tiles 256 columns wide: 4 x 2 (512 threads,
// two waves per SIMD, 64 x 128 or 32 x 128 per wave), so that the matrix pipe stays fed while one
// wave of a SIMD sits at the barrier or waits for LDS; the workgroup takes the whole LDS of a
// compute unit.  Tiles of 128 x 128: 2 x 2 (256 threads, 64 x 64 per wave) and half the LDS, so two
// workgroups share a compute unit and one's first loads and epilogue run under the other's main
// loop -- for launches whose tiles are short (few slabs) or few.
constexpr int kWavesN = 2;
constexpr int waves_m_of(int bn) { return bn == 128 ? 2 : 4; }
constexpr int threads_of(int bn) { return 64 * waves_m_of(bn) * kWavesN; }
constexpr int kThreads = threads_of(256);  // workgroup size of the stand-alone bias-gradient kernel
// The first kLoadWaves waves of a workgroup request the slabs.  The SIMD issues from its
// oldest wave first, so with two waves per SIMD the younger one falls behind; leaving the
// loads (which can block at a full load queue) to the older waves evens the two out.
constexpr int kLoadWaves = 4;
constexpr int kLoaders = 64 * kLoadWaves;
constexpr int kRowsPerPass = kLoaders / 8;  // KC slabs: rows covered by one 16-byte load of every loading thread
constexpr int kSlabBytes = 128;  // contraction bytes per row per slab
constexpr int kGroupM = 4;       // row tiles that share a column tile consecutively (an XCD then runs 4 x 8 tiles at a time)

enum Shape { kKC = 0, kMC = 1 };
enum Ragged { kRaggedRows = 0, kRaggedK = 1 };

// ---- element traits ---------------------------------------------------------
template <typename T> struct Elem;

// The 16-bit types use the 16 x 16 x 32 MFMA (4 accumulator registers per block): for the same
// flops it moves half as many accumulator registers as 32 x 32 x 16, and under the chip's
// power limit that buys clock.  fp32 uses 32 x 32 x 2.
template <> struct Elem<__bf16> {
    static constexpr int kPerChunk = 8;
    static constexpr int kBlk = 16;  // rows and columns of one MFMA block
    typedef f32x4 Acc;
    __device__ static __forceinline__ void mma(Acc &acc, const u32x4 &p, const u32x4 &q) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, p), __builtin_bit_cast(bf16x8, q),
                                                      acc, 0, 0, 0);
    }
    __device__ static __forceinline__ float to_float(__bf16 v) { return (float)v; }
};

template <> struct Elem<_Float16> {
    static constexpr int kPerChunk = 8;
    static constexpr int kBlk = 16;
    typedef f32x4 Acc;
    __device__ static __forceinline__ void mma(Acc &acc, const u32x4 &p, const u32x4 &q) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, p), __builtin_bit_cast(f16x8, q), acc,
                                                     0, 0, 0);
    }
};

template <> struct Elem<float> {
    static constexpr int kPerChunk = 4;
    static constexpr int kBlk = 32;
    typedef f32x16 Acc;
    __device__ static __forceinline__ void mma(Acc &acc, const u32x4 &p, const u32x4 &q) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(p[j]), __uint_as_float(q[j]), acc, 0, 0, 0);
    }
};

// erf by Abramowitz & Stegun 7.1.26 (|error| <= 1.5e-7): a reciprocal, an exponential and
// five multiply-adds instead of the library routine's branches.  The same exponential,
// exp(-x^2/2), is the Gaussian of GELU's derivative.
struct GeluTerms {
    float cdf;  // Phi(x) = 0.5 (1 + erf(x / sqrt 2))
    float pdf;  // phi(x) = exp(-x^2 / 2) / sqrt(2 pi)
};
__device__ __forceinline__ GeluTerms gelu_terms(float x) {
    const float z = fabsf(x) * 0.70710678118654752440f;
    const float t = __builtin_amdgcn_rcpf(1.f + 0.3275911f * z);
    const float e = __expf(-z * z);
    const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
    const float erf_abs = 1.f - poly * e;
    const float half_erf = 0.5f * (x < 0.f ? -erf_abs : erf_abs);
    return GeluTerms{0.5f + half_erf, 0.39894228040143267794f * e};
}

// Phi(x) - 1/2 for results that are rounded to 16 bits: an odd polynomial of degree 17 in x
// clamped to [-4.5, 4.5] (least-maximum-error fit, scaled to reach exactly 1/2 at the ends),
// |error| <= 4e-5, i.e. a hundredth of a bfloat16 rounding step -- 12 multiply-adds and two
// clamps, no reciprocal and no exponential (those run at a quarter of the multiply-add rate,
// and the activation is the only arithmetic in the epilogue that is not hidden behind loads).
__device__ __forceinline__ float cdf_minus_half_16bit(float x) {
    const float xc = __builtin_amdgcn_fmed3f(x, -4.5f, 4.5f);
    const float u = xc * xc;
    float r = 3.836310436e-11f;
    r = fmaf(r, u, -4.027055578e-09f);
    r = fmaf(r, u, 1.854241845e-07f);
    r = fmaf(r, u, -4.973333034e-06f);
    r = fmaf(r, u, 8.740126214e-05f);
    r = fmaf(r, u, -1.077337773e-03f);
    r = fmaf(r, u, 9.730750695e-03f);
    r = fmaf(r, u, -6.624028832e-02f);
    r = fmaf(r, u, 3.988564312e-01f);
    return __builtin_amdgcn_fmed3f(xc * r, -0.5f, 0.5f);
}

// GELU'(x) = Phi(x) + x phi(x) for results that are rounded to 16 bits: 1/2 plus an odd polynomial of
// degree 19 in x clamped to [-4.5, 4.5] (least-maximum-error fit; beyond the clamp the value stays
// within 7e-5 of the limits 0 and 1), |error| <= 6e-5 for |x| <= 3.5 and <= 1.4e-4 up to the clamp in
// single precision -- a fiftieth of a bfloat16 rounding step of the result (a seventh of a float16
// one, against a 2e-2 parity tolerance for both); 10 multiply-adds, one
// multiply and one clamp, no exponential (Phi - 1/2 from the polynomial above plus the Gaussian took
// 12 multiply-adds and an exponential, which issues at a quarter of the rate).
__device__ __forceinline__ float gelu_grad_16bit(float x) {
    const float xc = __builtin_amdgcn_fmed3f(x, -4.5f, 4.5f);
    const float u = xc * xc;
    float r = -2.210802284e-11f;
    r = fmaf(r, u, 2.521317906e-09f);
    r = fmaf(r, u, -1.268052924e-07f);
    r = fmaf(r, u, 3.721932329e-06f);
    r = fmaf(r, u, -7.122190070e-05f);
    r = fmaf(r, u, 9.405411684e-04f);
    r = fmaf(r, u, -8.815853635e-03f);
    r = fmaf(r, u, 5.860928472e-02f);
    r = fmaf(r, u, -2.649256521e-01f);
    r = fmaf(r, u, 7.976261318e-01f);
    // (the clamp drops a NaN; x * 0 puts it back, and gives NaN for an infinite pre-activation as
    // Phi(x) + x phi(x) evaluated literally does: a forward that overflowed still shows in the gradients)
    return fmaf(x, 0.f, fmaf(xc, r, 0.5f));
}

// Activation code inside the kernels only: exact GELU with the erf formula whatever the element type
// (FMOE_ACT_GELU takes the polynomials when the result is rounded to 16 bits).
constexpr int kActGeluErf = 3;

// kNarrow: the result is rounded to a 16-bit type
template <bool kNarrow> __device__ __forceinline__ float apply_act(float x, int act) {
    if (act == FMOE_ACT_RELU) return x > 0.f ? x : 0.f;
    if (act == FMOE_ACT_GELU || act == kActGeluErf) {
        if (kNarrow && act == FMOE_ACT_GELU) return fmaf(x, cdf_minus_half_16bit(x), 0.5f * x);
        return x * gelu_terms(x).cdf;
    }
    return x;
}

template <bool kNarrow> __device__ __forceinline__ float act_grad(float x, int act) {
    if (act == FMOE_ACT_RELU) return x > 0.f ? 1.f : 0.f;
    if (act == FMOE_ACT_GELU || act == kActGeluErf) {
        if (kNarrow && act == FMOE_ACT_GELU) return gelu_grad_16bit(x);
        const GeluTerms g = gelu_terms(x);
        return g.cdf + x * g.pdf;
    }
    return 1.f;
}

// ---- kernel arguments -------------------------------------------------------
struct GemmParams {
    const void *P;     // column operand (supplies C's columns)
    const void *Q;     // row operand (supplies C's rows)
    void *C;
    const void *bias;  // per expert [n_cols] or null
    void *bias_grad;   // ragged-K only: per expert [n_rows] column sums of Q (the output gradient), or null
    void *aux;         // see Epilogue
    int64_t ldp, ldq, ldc;      // leading dimensions in elements
    int64_t p_expert_stride;    // elements between two experts' P (0: P is row-indexed like Q)
    int64_t c_expert_stride;    // ragged-K: elements between two experts' C
    int64_t bias_expert_stride;
    int32_t n_cols;    // C columns = valid extent of P
    int32_t n_rows;    // ragged-K: C rows per expert = valid extent of Q
    int32_t k_extent;  // ragged-rows: contraction length
    int32_t tiles_n, tiles_m, total_tiles;
    int32_t activation;
    int32_t accumulate_first;  // ragged-K: expert 0 of the table adds to C
    int32_t epilogue;          // Epilogue, read by the any-shape kernel only
    // Ragged rows with a [row][contraction] row operand (the forward product) only: when q_row_index
    // is set, row r of the expert-sorted order is read from row q_row_index[r] / q_index_div of Q
    // (the token matrix, q_total_rows rows) instead of row r -- the local scatter happens in the
    // loader and the sorted copy of the input is never written.
    const int64_t *q_row_index;
    int64_t q_index_div, q_total_rows;
    // n / q_index_div for 0 <= n < 2^31 as umulhi(n, q_div_mul) >> q_div_shift (q_div_shift < 0: divisor 1);
    // filled in by set_row_index_divisor()
    uint32_t q_div_mul;
    int32_t q_div_shift;
    // Ragged rows only.  The tiles beyond the last whole round of the chip (tiles main_tiles ..
    // total_tiles - 1 of the logical order) can be split along the contraction: k_split
    // workgroups compute split_slabs slabs each and leave their fp32 accumulators in split_ws;
    // split_reduce_kernel then adds the parts of every tile in ascending order into part 0, and a
    // second launch of this kernel (fixup != 0, one wave per workgroup) loads the sums and runs
    // the epilogue.  k_split == 1: main_tiles == total_tiles.
    float *split_ws;
    int32_t main_tiles, k_split, split_slabs, fixup;
    // Segments from a table in device memory (segtab layout) instead of `tab`: the launch is sized
    // for the most tiles the table can describe, the kernel reads the real counts.  tab.n is then
    // the expert count (any number), tab.first_expert 0, and nothing is split.
    const int32_t *dev_tab;
    int32_t dev_map_off;       // offset (in int32) of the tile map for this launch's tile height
    // Device table and a caller's workspace for split tail tiles: dev_cus > 0 makes every workgroup plan
    // the tail split itself from the table's tile count, for dev_cus compute units (host only: dev_split_ws,
    // the workspace of at least dev_cus tiles of fp32 accumulators, copied to split_ws for the launch)
    int32_t dev_cus;
    float *dev_split_ws;
    int64_t dev_rows_cap;      // host only: rows the device table was laid out for
    int32_t block_m, block_n;  // host only: tile height the segment table was built for (256 or 128) and tile width
    int32_t profile_class;     // host only: ProfileClass of this launch
    double profile_work;       // host only: flop of this launch
    SegmentTable tab;
};

// Division of a 31-bit number by d through a multiplication: with s = ceil(log2 d) and
// m = floor(2^(31+s) / d) + 1 (which fits 32 bits for d >= 2), floor(n * m / 2^(31+s)) = floor(n / d) for
// every 0 <= n < 2^31, because the excess m d - 2^(31+s) is at most d <= 2^s, so the error term
// n (m d - 2^(31+s)) / (d 2^(31+s)) stays below 1 / d.
inline void set_row_index_divisor(GemmParams &prm, int64_t divisor) {
    prm.q_index_div = divisor;
    if (divisor <= 1) { prm.q_div_mul = 0; prm.q_div_shift = -1; return; }
    int s = 0;
    while (((int64_t)1 << s) < divisor) ++s;
    prm.q_div_mul = (uint32_t)((((uint64_t)1 << (31 + s)) / (uint64_t)divisor) + 1);
    prm.q_div_shift = s - 1;   // after the multiply-high's shift by 32
}

// How the tiles of a ragged-rows launch are spread over the chip.  One workgroup occupies a
// compute unit (two 128 x 128 workgroups share one, and then share its matrix pipe), so `total`
// tiles run in total / cus rounds and a last, partial round costs as much as a whole one.  When
// that last round fills at most half the chip, its tiles are split along the contraction into
// k_split parts (as many as fit the idle units, at most 8, at least 16 slabs each) -- provided
// that shortens the round by more than the partial sums' round trip through memory costs.
// slab_weight is the matrix-pipe time of a slab in units of a 16-bit slab's (2 for fp32: the same
// 128 bytes per row hold half the elements, each at a quarter of the rate).  Evaluated on the host
// for launches over host counts and by every workgroup for launches over a device table (where
// only the device knows the tile count).
constexpr int kMaxSplit = 8;
struct TailSplit {
    int main_tiles, k_split, split_slabs;
};
__host__ __device__ inline TailSplit plan_tail_split(int total, int n_slabs, int cus, int slab_weight = 1) {
    TailSplit p{total, 1, n_slabs};
    const int tail = total % cus;
    if (tail == 0 || tail * 2 > cus) return p;
    int f = cus / tail < kMaxSplit ? cus / tail : kMaxSplit;
    f = n_slabs * slab_weight / 16 < f ? n_slabs * slab_weight / 16 : f;
    if (f < 2) return p;
    const int per_part = (n_slabs + f - 1) / f;
    // the reduction and the second launch cost about as much as 40 (16-bit) slabs of one tile
    if ((n_slabs - per_part) * slab_weight < 40) return p;
    p.split_slabs = per_part;
    p.k_split = (n_slabs + p.split_slabs - 1) / p.split_slabs;  // no empty part
    p.main_tiles = total - tail;
    return p;
}
// whether any tile count at all makes plan_tail_split split a contraction of n_slabs slabs
inline bool tail_split_possible(int n_slabs, int slab_weight = 1) {
    const int f = n_slabs * slab_weight / 16 < kMaxSplit ? n_slabs * slab_weight / 16 : kMaxSplit;
    return f >= 2 && (n_slabs - (n_slabs + f - 1) / f) * slab_weight >= 40;
}
template <typename T> constexpr int slab_weight_of() { return sizeof(T) == 4 ? 2 : 1; }

// KC slabs: 16-byte chunk c of row r is stored at chunk c ^ swz(r).
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }
// MC slabs of 16-bit elements: chunk c of contraction row k is stored at
// c ^ ((k % 4) * 4 + (k / 8 % 2) * 2).  A transposing read of 32 lanes touches two blocks of
// 4 k rows x 2 chunks, 8 k rows apart; rows are a multiple of 256 B apart, so without the
// swizzle they would share banks -- with it the 16 chunks fall on the 16 distinct 16-byte
// positions of the 256-byte bank cycle.
template <typename T> __device__ __forceinline__ int mc_swz(int k) {
    return sizeof(T) == 2 ? ((k & 3) << 2) | (((k >> 3) & 1) << 1) : 0;
}

// ---- the kernel ---------------------------------------------------------------
template <typename T, int BM, int BN, int PSHAPE, int QSHAPE, int RAGGED, int EPI>
__global__ __launch_bounds__(threads_of(BN)) void grouped_gemm_kernel(const GemmParams prm) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub
    constexpr int kWavesM = waves_m_of(BN), kWaves = kWavesM * kWavesN;
    constexpr int kThreads = threads_of(BN);
    static_assert(kWaves >= kLoadWaves && (kWaves & (kWaves - 1)) == 0, "wave layout");
    constexpr int CE = Elem<T>::kPerChunk;           // elements per 16-byte chunk
    constexpr int BKE = kSlabBytes / (int)sizeof(T); // elements per slab row
    constexpr int WM = BM / kWavesM, WN = BN / kWavesN;  // wave tile
    constexpr int MB = Elem<T>::kBlk;                // MFMA block edge
    constexpr int TI = WN / MB, TJ = WM / MB;        // MFMA blocks per wave (cols, rows)
    constexpr int kAccRegs = MB * MB / 64;           // accumulator registers per block
    constexpr int kChunksPerStep = 64 / MB;          // 16-byte contraction chunks one MFMA step consumes per row
    constexpr int NP = BN * 8 / kLoaders;            // 16-byte chunks per loading thread per slab
    constexpr int NQ = BM * 8 / kLoaders;
    constexpr int P_BYTES = BN * kSlabBytes, Q_BYTES = BM * kSlabBytes;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    // -- which tile ------------------------------------------------------------
    // Workgroup b runs on XCD b % 8 (each XCD has its own L2).  Ragged rows: tiles cost the
    // same, so every XCD takes a contiguous eighth of the logical tile order.  Ragged K: a
    // tile costs as much as its expert has rows, so every XCD takes a contiguous eighth of
    // EACH expert's tiles instead -- skewed routing then loads the XCDs evenly.
    int ei, mt, nt;
    int split_part = -1;   // >= 0: this workgroup computes that part of the contraction of a tail tile
    int tail_index = 0;    // index of a tail tile among the tail tiles
    const bool fixup = RAGGED == kRaggedRows && prm.fixup != 0;
    int k_split = prm.k_split, split_slabs = prm.split_slabs;  // (a launch over a device table plans them below)
    // the device table is read-only while the kernel runs and addressed uniformly: scalar loads
    typedef const int32_t __attribute__((address_space(4))) *DevTab;
    const DevTab dtab = (DevTab)(uintptr_t)prm.dev_tab;
    const bool dev = prm.dev_tab != nullptr;
    int seg_lo, seg_hi;
    {
        int tm_total, rem;
        if (RAGGED == kRaggedRows) {
            int L;
            int main_tiles = prm.main_tiles, total_tiles = prm.total_tiles;
            if (dev) {
                tm_total = dtab[BM == 256 ? segtab::kTiles256 : segtab::kTiles128];
                main_tiles = total_tiles = tm_total * prm.tiles_n;
                if (prm.dev_cus > 0) {
                    const TailSplit ts = plan_tail_split(total_tiles, (prm.k_extent + BKE - 1) / BKE, prm.dev_cus, slab_weight_of<T>());
                    main_tiles = ts.main_tiles;
                    k_split = ts.k_split;
                    split_slabs = ts.split_slabs;
                }
            } else {
                tm_total = prm.tab.tile[prm.tab.n];
            }
            const int main_grid = (main_tiles + 7) & ~7;
            if (fixup) {
                tail_index = blockIdx.x / kWaves;  // one one-wave workgroup per wave of a tail tile
                // (device table: the launch was sized for the most tail tiles there can be)
                if (dev && (k_split == 1 || tail_index >= total_tiles - main_tiles)) return;
                L = main_tiles + tail_index;
            } else if ((int)blockIdx.x < main_grid) {
                const int per_xcd = main_grid >> 3;
                L = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
                if (L >= main_tiles) return;
            } else {
                const int u = blockIdx.x - main_grid, n_tail = total_tiles - main_tiles;
                if (dev && (k_split == 1 || u >= n_tail * k_split)) return;  // the launch was sized for an upper bound
                split_part = u / n_tail;
                tail_index = u - split_part * n_tail;
                L = main_tiles + tail_index;
            }
            rem = L;
            ei = 0;
        } else {
            const int tpe = prm.tiles_m * prm.tiles_n;
            const int share = (tpe + 7) >> 3;  // tiles of one expert per XCD
            const int i = blockIdx.x >> 3;
            tm_total = prm.tiles_m;
            ei = i / share;
            rem = (blockIdx.x & 7) * share + (i - ei * share);
            if (ei >= prm.tab.n || rem >= tpe) return;
        }
        const int gspan = kGroupM * prm.tiles_n;
        const int grp = rem / gspan;
        const int first_m = grp * kGroupM;
        const int gsz = min(kGroupM, tm_total - first_m);
        const int in_grp = rem - grp * gspan;
        mt = first_m + in_grp % gsz;
        nt = in_grp / gsz;
        if (RAGGED == kRaggedRows) {
            if (dev) {
                // {expert, first row, rows} of row tile mt
                // (the map's offset is known to the host, so this load waits for the tile count only)
                typedef int i32x4 __attribute__((ext_vector_type(4)));
                typedef const i32x4 __attribute__((address_space(4))) *DevTab4;
                const i32x4 entry = *(DevTab4)(dtab + prm.dev_map_off + 4 * mt);
                ei = entry[0];
                seg_lo = entry[1];
                seg_hi = seg_lo + entry[2];
            } else {
                int lo = 0, hi = prm.tab.n;  // tile[lo] <= mt < tile[hi]
                while (hi - lo > 1) {
                    const int mid = (lo + hi) >> 1;
                    if (prm.tab.tile[mid] <= mt) lo = mid; else hi = mid;
                }
                ei = lo;
            }
        }
    }
    const int expert = prm.tab.first_expert + ei;
    if (RAGGED == kRaggedK && dev) {
        seg_lo = dtab[segtab::kHeader + ei];
        seg_hi = dtab[segtab::kHeader + ei + 1];
    } else if (!(RAGGED == kRaggedRows && dev)) {
        seg_lo = prm.tab.seg[ei];
        seg_hi = prm.tab.seg[ei + 1];
    }
    const int n0 = nt * BN;

    const T *Pb;
    const T *Qb;
    T *Cb;
    int p_valid, q_valid, K;
    int q_row0 = 0;
    const bool gather_q = RAGGED == kRaggedRows && QSHAPE == kKC && prm.q_row_index != nullptr;
    int64_t q_gather_bytes = 0;  // extent of the gathered matrix past this part's first contraction element
    int64_t aux_off;  // offset of this tile's origin inside C (and aux)
    if (RAGGED == kRaggedRows) {
        // (device table: seg_lo .. seg_hi are the rows of this very tile)
        const int row0 = dev ? seg_lo : seg_lo + (mt - prm.tab.tile[ei]) * BM;
        q_row0 = row0;
        q_valid = min(BM, seg_hi - row0);
        K = prm.k_extent;
        Qb = (const T *)prm.Q + (gather_q ? (int64_t)0 : (int64_t)row0 * prm.ldq);
        const T *Pe = (const T *)prm.P + (int64_t)expert * prm.p_expert_stride;
        Pb = (PSHAPE == kKC) ? Pe + (int64_t)n0 * prm.ldp : Pe + n0;
        aux_off = (int64_t)row0 * prm.ldc + n0;
        if (split_part >= 0) {  // this part's slabs only
            const int k_begin = split_part * split_slabs * BKE;
            K = max(0, min(K - k_begin, split_slabs * BKE));
            Qb += (QSHAPE == kKC) ? (int64_t)k_begin : (int64_t)k_begin * prm.ldq;
            q_gather_bytes = -(int64_t)k_begin * (int64_t)sizeof(T);
            Pb += (PSHAPE == kKC) ? (int64_t)k_begin : (int64_t)k_begin * prm.ldp;
        }
    } else {
        const int m0 = mt * BM;
        q_valid = min(BM, prm.n_rows - m0);
        K = seg_hi - seg_lo;
        Qb = (const T *)prm.Q + (int64_t)seg_lo * prm.ldq + m0;
        Pb = (const T *)prm.P + (int64_t)seg_lo * prm.ldp + n0;
        aux_off = (int64_t)expert * prm.c_expert_stride + (int64_t)m0 * prm.ldc + n0;
    }
    p_valid = min(BN, prm.n_cols - n0);
    Cb = (T *)prm.C + aux_off;

    const int t = threadIdx.x;
    // a fixup launch runs one wave per workgroup; it stands in for wave blockIdx.x % kWaves of the tile's workgroup
    const int lane = t & 63, wave = fixup ? (int)(blockIdx.x % kWaves) : t >> 6;
    const int lb = lane & (MB - 1), hq = lane / MB;  // row inside an MFMA block, contraction chunk inside a step
    const int wave_m0 = (wave / kWavesN) * WM, wave_n0 = (wave % kWavesN) * WN;

    // An expert without rows has a zero weight gradient (and bias gradient): write the
    // tile with plain coalesced stores and skip the whole pipeline.
    if constexpr (RAGGED == kRaggedK) {
        if (K == 0) {
            constexpr int kChunksPerRow = BN / CE;
            for (int q = t; q < BM * kChunksPerRow; q += kThreads) {
                const int r = q / kChunksPerRow, c = q % kChunksPerRow;
                if (r < q_valid && c * CE < p_valid) *(u32x4 *)(Cb + (int64_t)r * prm.ldc + c * CE) = u32x4{0, 0, 0, 0};
            }
            if (prm.bias_grad != nullptr && nt == 0 && t < q_valid)
                ((T *)prm.bias_grad)[(int64_t)expert * prm.n_rows + mt * BM + t] = (T)0.f;
            return;
        }
    }

    // -- global -> LDS staging ------------------------------------------------------
    // Slabs go from memory straight into LDS (buffer_load ... lds: lane i of a wave lands
    // at base + 16 i).  An offset at or beyond the buffer resource's size returns zeros, so
    // rows outside the tile and the contraction tail need no branch -- their offset is
    // replaced by kOutOfRange and the lanes land as zeros.
    //
    // LDS holds three buffers for P slabs followed by two for Q slabs (160 KiB at 256 x 256).
    // While slab s is computed from, slab s+1 is complete or landing, the P part of slab s+2
    // is requested at the start of slab s and its Q part right after the barrier that ends
    // slab s: the loads are spread over the slab (a burst of them would fill the load
    // queue and block the MFMAs behind it) and the P loads have more than a slab to land.
    constexpr uint32_t kOutOfRange = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format
    constexpr int P_CPR = BN / CE, P_KPI = kLoaders / P_CPR;  // MC: chunks per k row, k rows per pass
    constexpr int Q_CPR = BM / CE, Q_KPI = kLoaders / Q_CPR;
    constexpr int kPassBytes = kLoaders * 16;  // LDS bytes filled by one 16-byte load of every loading thread
    constexpr int kPBufs = 3;
    constexpr int Q_BASE = kPBufs * P_BYTES;

    // Slot q = it*kLoaders + t of a slab is filled by thread t < kLoaders in pass it, so a wave fills
    // 1 KiB of consecutive LDS per load.  The swizzle is applied on the memory side: the
    // thread fetches the chunk that belongs in its slot.
    //   KC: slot q is row q/8, position q%8, and holds chunk (q%8) ^ swz(row)
    //   MC: slot q is contraction row q/CPR, position q%CPR, and holds chunk (q%CPR) ^ mc_swz(k)
    uint32_t p_voff[NP], q_voff[NQ];
    int p_kc_chunk = 0, q_kc_chunk = 0;  // KC: logical chunk of this thread (same in every pass)
    if (PSHAPE == kKC) {
        const int r = t >> 3;
        p_kc_chunk = (t & 7) ^ swz(r);
#pragma unroll
        for (int it = 0; it < NP; ++it)
            p_voff[it] = (it * kRowsPerPass + r < p_valid)
                             ? (uint32_t)(((int64_t)(it * kRowsPerPass + r) * prm.ldp + p_kc_chunk * CE) * sizeof(T))
                             : kOutOfRange;
    } else {
        const int kk = t / P_CPR;
#pragma unroll
        for (int it = 0; it < NP; ++it) {
            const int c = (t % P_CPR) ^ mc_swz<T>(it * P_KPI + kk);
            p_voff[it] = (c * CE < p_valid)
                             ? (uint32_t)(((int64_t)(it * P_KPI + kk) * prm.ldp + c * CE) * sizeof(T))
                             : kOutOfRange;
        }
    }
    if (QSHAPE == kKC) {
        const int r = t >> 3;
        q_kc_chunk = (t & 7) ^ swz(r);
        if (gather_q) {
            // the resource covers the whole token matrix (less than 2 GiB, checked by the host) from this
            // part's first contraction element on; a row index outside it reads as zeros
            q_gather_bytes += prm.q_total_rows * prm.ldq * (int64_t)sizeof(T);
#pragma unroll
            for (int it = 0; it < NQ; ++it) {
                const int row = it * kRowsPerPass + r;
                int64_t src = -1;
                if (row < q_valid && t < kLoaders) {
                    // slot indices fit 31 bits (checked by the host), so idx / q_index_div is a multiply-high and
                    // a shift by constants the host derived from the divisor (a 64-bit division takes hundreds
                    // of instructions, and eight of them stood between a tile's start and its first loads)
                    const int64_t idx = prm.q_row_index[q_row0 + row];
                    if (idx >= 0 && idx <= (int64_t)INT32_MAX)
                        src = prm.q_div_shift < 0 ? idx : (int64_t)(__umulhi((uint32_t)idx, prm.q_div_mul) >> prm.q_div_shift);
                }
                q_voff[it] = (src >= 0 && src < prm.q_total_rows)
                                 ? (uint32_t)((src * prm.ldq + q_kc_chunk * CE) * (int64_t)sizeof(T))
                                 : kOutOfRange;
            }
        } else {
#pragma unroll
            for (int it = 0; it < NQ; ++it)
                q_voff[it] = (it * kRowsPerPass + r < q_valid)
                                 ? (uint32_t)(((int64_t)(it * kRowsPerPass + r) * prm.ldq + q_kc_chunk * CE) * sizeof(T))
                                 : kOutOfRange;
        }
    } else {
        const int kk = t / Q_CPR;
#pragma unroll
        for (int it = 0; it < NQ; ++it) {
            const int c = (t % Q_CPR) ^ mc_swz<T>(it * Q_KPI + kk);
            q_voff[it] = (c * CE < q_valid)
                             ? (uint32_t)(((int64_t)(it * Q_KPI + kk) * prm.ldq + c * CE) * sizeof(T))
                             : kOutOfRange;
        }
    }

    // With an MC slab the fragments are read by ds_read_b64_tr_b16, and the compiler puts a
    // full vmcnt(0) wait between a direct-to-LDS load and any such read that follows it
    // (it cannot tell the LDS buffers apart), which would serialise the pipeline.  For
    // those products the load is emitted as inline assembly, which the compiler does not
    // track; the waits that are needed (before the barriers) are written out by hand.
    constexpr bool kDmaAsm = (PSHAPE == kMC || QSHAPE == kMC);
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)smem;
    const uint32_t wave_u = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    auto dma_asm = [&](const T *origin, int64_t bytes, uint32_t lds_off, uint32_t voff) {
        const uint64_t a = (uint64_t)origin;
        i32x4 rs;
        rs[0] = (int)(uint32_t)a;
        rs[1] = (int)((uint32_t)(a >> 32) & 0xffffu);
        rs[2] = (int)bytes;
        rs[3] = kRsrcFlags;
        rs[0] = __builtin_amdgcn_readfirstlane(rs[0]);
        rs[1] = __builtin_amdgcn_readfirstlane(rs[1]);
        rs[2] = __builtin_amdgcn_readfirstlane(rs[2]);
        const uint32_t lds_addr = __builtin_amdgcn_readfirstlane(lds_base + lds_off);
        asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(rs)
                     : "memory", "m0");
    };

    // One operand's part of the slab that starts at contraction index k0, into LDS offset
    // lds_off.  KC: the resource starts at contraction index k0 of the tile's first row and
    // the chunk is dropped when it lies past K.  MC: the resource starts at contraction row
    // k0 and is exactly as long as the rows that remain, so rows past K read as zero.
    auto issue_part = [&](auto shape_tag, const T *tile, int64_t ld, int kc_chunk, const uint32_t *voff, auto n_tag, int k0,
                          uint32_t lds_off, int it_lo = 0, int it_hi = 1 << 20, int64_t kc_extent = (int64_t)1 << 40) {
        constexpr int SHAPE = decltype(shape_tag)::value;
        constexpr int N = decltype(n_tag)::value;
        const int k_left = K - k0;  // <= 0 past the end: everything reads as zero
        const T *origin = (SHAPE == kKC) ? tile + k0 : tile + (int64_t)k0 * ld;
        // KC: the rows of a tile lie within 2 GiB of its origin; gathered rows within kc_extent bytes of the matrix
        int64_t bytes = (SHAPE == kKC) ? kc_extent - (int64_t)k0 * (int64_t)sizeof(T)
                                       : (int64_t)k_left * ld * (int64_t)sizeof(T);
        bytes = bytes < 0 ? 0 : (bytes > (int64_t)kOutOfRange ? (int64_t)kOutOfRange : bytes);
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(origin), 0, (int)bytes, kRsrcFlags);
        // sign bit of (k_left - 1 - first k of the chunk): set exactly when the chunk starts past K
        const uint32_t past = (SHAPE == kKC) ? ((uint32_t)(k_left - 1 - kc_chunk * CE) & kOutOfRange) : 0u;
#pragma unroll
        for (int it = 0; it < N; ++it) {
            if (it < it_lo || it >= it_hi) continue;
            if constexpr (kDmaAsm)
                dma_asm(origin, bytes, lds_off + wave_u * 1024 + it * kPassBytes, voff[it] | past);
            else
                __builtin_amdgcn_raw_ptr_buffer_load_lds(
                    rsrc, (__attribute__((address_space(3))) void *)(smem + lds_off + wave * 1024 + it * kPassBytes), 16,
                    voff[it] | past, 0, 0, 0);
        }
    };
    auto issue_p = [&](int k0, int buf, int it_lo = 0, int it_hi = 1 << 20) {
        issue_part(std::integral_constant<int, PSHAPE>{}, Pb, prm.ldp, p_kc_chunk, p_voff, std::integral_constant<int, NP>{}, k0,
                   (uint32_t)(buf * P_BYTES), it_lo, it_hi);
    };
    auto issue_q = [&](int k0, int buf) {
        issue_part(std::integral_constant<int, QSHAPE>{}, Qb, prm.ldq, q_kc_chunk, q_voff, std::integral_constant<int, NQ>{}, k0,
                   (uint32_t)(Q_BASE + buf * Q_BYTES), 0, 1 << 20, gather_q ? q_gather_bytes : (int64_t)1 << 40);
    };

    // Data-grad with the activation derivative, 16-bit types: the tile of saved
    // pre-activations that the epilogue needs (BM rows x 512 bytes) is requested in the load
    // slots of the last two slabs, whose own loads would only fetch zeros past the end of
    // the contraction -- 64 rows (one P buffer's worth) per slot, parts 0 and 1 in the P slots,
    // parts 2 and 3 (256-row tiles) in the Q slots -- so it lands while the last MFMAs run
    // instead of after them, when every workgroup of the round asks memory at once.
    // Slot q of a part is row q/32, position q%32, and holds chunk (q%32) ^ (row%16).
    constexpr bool kAuxPrefetch = EPI == kEpiDAct && sizeof(T) == 2 && kDmaAsm && BN == 256;
    constexpr int kAuxParts = BM / 64;
    const T *aux_tile = (const T *)prm.aux + aux_off;
    auto issue_aux = [&](int part, uint32_t lds_off) {
        if constexpr (kAuxPrefetch) {
#pragma unroll
            for (int it = 0; it < NP; ++it) {
                const int rip = it * 8 + (t >> 5);              // row inside the part
                const int row = part * 64 + rip;
                const int c = (t & 31) ^ (rip & 15);
                const bool ok = row < q_valid && c * CE < p_valid;
                const uint32_t voff = ok ? (uint32_t)(((int64_t)row * prm.ldc + c * CE) * sizeof(T)) : kOutOfRange;
                dma_asm(aux_tile, (int64_t)kOutOfRange, lds_off + wave_u * 1024 + it * kPassBytes, voff);
            }
        }
    };

    // Bias gradient (weight-gradient product only): the workgroups of the first column
    // tile also add up the rows of the Q slabs they stage, i.e. the column sums of the
    // output gradient over the expert's rows.  Every thread keeps the sums of the CE
    // columns of its chunk; they are combined across threads after the main loop.
    float bsum[CE];
#pragma unroll
    for (int j = 0; j < CE; ++j) bsum[j] = 0.f;
    auto add_chunk = [&](const u32x4 &v) {
        if (sizeof(T) == 4) {
#pragma unroll
            for (int j = 0; j < 4; ++j) bsum[j] += __uint_as_float(v[j]);
        } else if (std::is_same<T, __bf16>::value) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                bsum[2 * j] += __uint_as_float(v[j] << 16);
                bsum[2 * j + 1] += __uint_as_float(v[j] & 0xffff0000u);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                bsum[2 * j] += (float)__builtin_bit_cast(_Float16, (uint16_t)(v[j] & 0xffffu));
                bsum[2 * j + 1] += (float)__builtin_bit_cast(_Float16, (uint16_t)(v[j] >> 16));
            }
        }
    };
    // adds up this thread's share of the chunks in Q buffer `buf` (after they have landed):
    // slots t, t + kThreads, ... -- the same column chunk in every one of them
    constexpr int kBiasPasses = BM * 8 / kThreads, kBiasKPI = kThreads / Q_CPR;
    auto add_q_chunks = [&](int buf) {
        const unsigned char *sq = smem + Q_BASE + buf * Q_BYTES + t * 16;
#pragma unroll
        for (int it = 0; it < kBiasPasses; ++it) add_chunk(*(const u32x4 *)(sq + it * kThreads * 16));
    };

    // -- fragments ---------------------------------------------------------------
    // A fragment is the 16 bytes a lane feeds to the MFMA for one block of MB rows and one
    // contraction step (64 bytes of the slab row for 16-bit types, 32 for fp32):
    // row = block row lb, contraction chunk = kChunksPerStep * step + hq.
    auto frag = [&](const unsigned char *slab, int shape, int extent, int r0, int ks) -> u32x4 {
        if (shape == kKC) {
            const int row = r0 + lb;
            const int chunk = ks * kChunksPerStep + hq;
            return *(const u32x4 *)(slab + row * kSlabBytes + ((chunk ^ swz(row)) << 4));
        }
        u32x4 out;
        if constexpr (sizeof(T) == 4) {
            const int row = r0 + lb;
            const uint32_t *s = (const uint32_t *)slab;
#pragma unroll
            for (int j = 0; j < 4; ++j) out[j] = s[(ks * 8 + hq * 4 + j) * extent + row];
        } else {
            // ds_read_b64_tr_b16: a 16-lane group reads a 4(k) x 16(row) block of 16-bit
            // elements, lane s of the group pointing at row-of-k s/4, columns 4*(s%4)..+3,
            // and receives column s of the block with its 4 k values.  Group g takes the 16
            // rows of the MFMA block at contraction indices 8g..8g+3 of the step; the
            // second read is 4 k further on.
            const int s16 = lane & 15;
            const int col = r0 + 4 * (s16 & 3);
            const int kb = ks * 32 + hq * 8 + (s16 >> 2);
            const int chunk = (col >> 3) ^ mc_swz<T>(kb);  // kb and kb + 4 swizzle alike
            const unsigned char *base = slab + chunk * 16 + (col & 7) * 2;
            typedef short s16x4 __attribute__((ext_vector_type(4)));
            typedef __attribute__((address_space(3))) s16x4 *lds_s16x4_ptr;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(base + kb * extent * 2));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(base + (kb + 4) * extent * 2));
            const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
            out = u32x4{l2[0], l2[1], h2[0], h2[1]};
        }
        return out;
    };

    typename Elem<T>::Acc acc[TI][TJ];
#pragma unroll
    for (int x = 0; x < TI; ++x)
#pragma unroll
        for (int y = 0; y < TJ; ++y)
#pragma unroll
            for (int r = 0; r < kAccRegs; ++r) acc[x][y][r] = 0.f;

    // Main loop, one basic block per slab, software-pipelined by hand.  A slab is worked
    // through in four phases.  fp32 (32 x 32 blocks): a phase is one contraction step over
    // all block columns.  16-bit (16 x 16 blocks): a phase is half the block columns of one
    // of the slab's two contraction steps, so the Q fragments are read every other phase.
    // P buffer pc holds slab s, pn slab s+1, pf_buf receives slab s+2; Q buffer s%2 holds
    // slab s.  Per slab:
    //   phase 0     : MFMAs of the phase, LDS reads of phase 1 between them
    //   phases 1..2 : MFMAs of the phase, LDS reads of the next one, and half of the P loads
    //                 of slab s+2 each
    //   wait        : until this wave's loads of slab s+1 have landed (the P loads of slab
    //                 s+2 stay in flight) and its reads of phase 3 have returned
    //   barrier     : slab s+1 is complete and nobody reads slab s any more
    //   phase 3     : its MFMAs (from fragments already in registers); the Q part of slab
    //                 s+2 is requested into the Q buffer of slab s and phase 0 of slab s+1
    //                 is read
    // so no LDS read is waited for at the top of an iteration, and a whole phase of MFMAs
    // covers the reads that follow the barrier (with part of phase 3 ahead of the barrier
    // the step measured 0.8 % slower).  Past the last slab the
    // loads return zeros and land in buffers nobody reads, which keeps the body branch-free.
    constexpr int kPhases = 4;
    constexpr int PF = (MB == 32) ? TI : TI / 2;                // block columns per phase
    constexpr int kPReadsPerFrag = (PSHAPE == kMC) ? (sizeof(T) == 2 ? 2 : 4) : 1;
    constexpr int kQReadsPerFrag = (QSHAPE == kMC) ? (sizeof(T) == 2 ? 2 : 4) : 1;
    constexpr int kMfma = PF * TJ * (sizeof(T) == 4 ? 4 : 1);   // MFMA instructions per phase
    constexpr int kReadsPerMfma = 1;  // a phase's reads go out early, one per MFMA; the remaining MFMAs follow
    static_assert(NP % 2 == 0 && NP / 2 <= kMfma, "the P loads of a slab go out in two halves, one load per MFMA");
    // phases that carry the two halves: phase 3 carries the Q loads, phase 0 is left to let
    // the load queue drain (0 and 1 measured 0.5 % slower per step, all in phase 0 1 %)
    constexpr int kPLoadPhaseA = 1, kPLoadPhaseB = 2;
    // contraction step, first block column, Q fragment buffer of a phase; does it start a step
    auto phase_ks = [](int ph) { return MB == 32 ? ph : ph >> 1; };
    auto phase_x0 = [](int ph) { return MB == 32 ? 0 : (ph & 1) * PF; };
    auto phase_qbuf = [](int ph) { return MB == 32 ? (ph & 1) : ((ph >> 1) & 1); };
    auto phase_reads_q = [](int ph) { return MB == 32 || (ph & 1) == 0; };
    auto phase_reads = [&](int ph) { return PF * kPReadsPerFrag + (phase_reads_q(ph) ? TJ * kQReadsPerFrag : 0); };

    const int n_slabs = (K + BKE - 1) / BKE;
    const bool aux_pref = kAuxPrefetch && n_slabs >= 2 && split_part < 0 && !fixup;  // both tail slabs exist
    u32x4 pf[2][PF], qf[2][TJ];
    // the fragments of phase ph, in the order its MFMAs (x outer, y inner) first need them
    auto read_phase = [&](int ph, const unsigned char *sp, const unsigned char *sq) {
        if (phase_reads_q(ph)) {
#pragma unroll
            for (int y = 0; y < TJ; ++y) qf[phase_qbuf(ph)][y] = frag(sq, QSHAPE, BM, wave_m0 + y * MB, phase_ks(ph));
        }
#pragma unroll
        for (int x = 0; x < PF; ++x) pf[ph & 1][x] = frag(sp, PSHAPE, BN, wave_n0 + (phase_x0(ph) + x) * MB, phase_ks(ph));
    };
    auto mma_phase = [&](int ph, int x_lo, int x_hi) {
#pragma unroll
        for (int x = x_lo; x < x_hi; ++x)
#pragma unroll
            for (int y = 0; y < TJ; ++y) Elem<T>::mma(acc[phase_x0(ph) + x][y], pf[ph & 1][x], qf[phase_qbuf(ph)][y]);
    };
    // s_waitcnt vmcnt(n) lgkmcnt(0): at most n of this wave's loads still in flight, all LDS reads done
    auto wait_loads = [&](auto n_tag) {
        constexpr int n = decltype(n_tag)::value;
        static_assert(n < 64, "vmcnt is a 6-bit field");
        __builtin_amdgcn_s_waitcnt(0x0070 | (n & 15) | ((n >> 4) << 14));
    };
    // LDS reads are complete (waited for above) when a wave arrives, so the barrier alone
    // orders them against the loads that overwrite the buffer afterwards
    auto slab_barrier = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };

    auto main_loop = [&](auto with_bias, auto loads_tag) {
        constexpr bool kBias = decltype(with_bias)::value;
        constexpr bool kLoads = decltype(loads_tag)::value;  // this wave requests slabs
        constexpr int kNoWait = 63;
        if constexpr (kLoads) {
            issue_p(0, 0);
            issue_q(0, 0);
            issue_p(BKE, 1);
            issue_q(BKE, 1);
        }
        __builtin_amdgcn_sched_barrier(0);
        wait_loads(std::integral_constant<int, kLoads ? NP + NQ : kNoWait>{});  // slab 0 has landed
        slab_barrier();
        if constexpr (kBias) add_q_chunks(0);
        read_phase(0, smem, smem + Q_BASE);
        __builtin_amdgcn_sched_barrier(0);

        int pc = 0;
        for (int s = 0; s < n_slabs; ++s) {
            const int pn = pc == kPBufs - 1 ? 0 : pc + 1;
            const int pf_buf = pn == kPBufs - 1 ? 0 : pn + 1;
            const unsigned char *sp = smem + pc * P_BYTES;
            const unsigned char *sq = smem + Q_BASE + (s & 1) * Q_BYTES;
#pragma unroll
            for (int ph = 0; ph + 1 < kPhases; ++ph) {
                if (kLoads && ph == kPLoadPhaseA) {
                    const int past_end = s + 2 - n_slabs;  // >= 0: slab s+2 does not exist
                    if (kAuxPrefetch && aux_pref && past_end >= 0) issue_aux(past_end, (uint32_t)(pf_buf * P_BYTES));
                    else issue_p((s + 2) * BKE, pf_buf, 0, NP / 2);
                }
                if (kLoads && ph == kPLoadPhaseB) {  // the second half of the P loads (the pre-activation part went out whole)
                    const int past_end = s + 2 - n_slabs;
                    if (!(kAuxPrefetch && aux_pref && past_end >= 0)) issue_p((s + 2) * BKE, pf_buf, NP / 2, NP);
                }
                read_phase(ph + 1, sp, sq);
                mma_phase(ph, 0, PF);
#pragma unroll
                for (int i = 0; i < kMfma; ++i) {
                    if (i * kReadsPerMfma < phase_reads(ph + 1)) __builtin_amdgcn_sched_group_barrier(0x100, kReadsPerMfma, 0);  // LDS reads
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                                       // one MFMA
                    if (kLoads && (ph == kPLoadPhaseA || ph == kPLoadPhaseB) && i < NP / 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one load
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            wait_loads(std::integral_constant<int, kLoads ? NP : kNoWait>{});  // everything but the P loads of slab s+2
            slab_barrier();
            if constexpr (kBias) add_q_chunks((s + 1) & 1);
            if constexpr (kLoads) {
                const int past_end = s + 2 - n_slabs;
                if (kAuxPrefetch && kAuxParts == 4 && aux_pref && past_end >= 0)
                    issue_aux(2 + past_end, (uint32_t)(Q_BASE + (s & 1) * Q_BYTES));
                else
                    issue_q((s + 2) * BKE, s & 1);
            }
            read_phase(0, smem + pn * P_BYTES, smem + Q_BASE + ((s + 1) & 1) * Q_BYTES);
            mma_phase(kPhases - 1, 0, PF);
            constexpr int kQLoadsPerMfma = (NQ + kMfma - 1) / kMfma;
#pragma unroll
            for (int i = 0; i < kMfma; ++i) {
                if (i * kReadsPerMfma < phase_reads(0)) __builtin_amdgcn_sched_group_barrier(0x100, kReadsPerMfma, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if (kLoads && i * kQLoadsPerMfma < NQ) __builtin_amdgcn_sched_group_barrier(0x020, kQLoadsPerMfma, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            pc = pn;
        }
        // the loads requested past the last slab (all out of range) must land before LDS is reused
        wait_loads(std::integral_constant<int, 0>{});
        slab_barrier();
    };
    auto run_loop = [&](auto with_bias) {
        if (wave_u < (uint32_t)kLoadWaves) main_loop(with_bias, std::true_type{});
        else main_loop(with_bias, std::false_type{});
    };
    bool want_bias = false;
    if constexpr (RAGGED == kRaggedK && QSHAPE == kMC) want_bias = prm.bias_grad != nullptr && nt == 0;
    if constexpr (RAGGED == kRaggedK && QSHAPE == kMC) {
        if (want_bias) run_loop(std::true_type{});
        else run_loop(std::false_type{});
    } else {
        if (!fixup) run_loop(std::false_type{});
    }

    // Split tail tiles.  Part p of tail tile i keeps its accumulators in
    // split_ws[(i * k_split + p) * BM * BN ...] as [float4 index j][thread], j running over
    // (block column, block row, quarter of the block's registers): every store and load
    // instruction of a wave covers 1 KiB of consecutive memory.
    if constexpr (RAGGED == kRaggedRows) {
        constexpr int kVecPerBlk = kAccRegs / 4;
        constexpr int64_t kTileVecs = (int64_t)BM * BN / 4;
        if (split_part >= 0) {
            f32x4 *dst = (f32x4 *)prm.split_ws + ((int64_t)tail_index * k_split + split_part) * kTileVecs + t;
#pragma unroll
            for (int x = 0; x < TI; ++x)
#pragma unroll
                for (int y = 0; y < TJ; ++y)
#pragma unroll
                    for (int v = 0; v < kVecPerBlk; ++v) {
                        const int j = (x * TJ + y) * kVecPerBlk + v;
                        f32x4 val;
#pragma unroll
                        for (int i = 0; i < 4; ++i) val[i] = acc[x][y][4 * v + i];
                        __builtin_nontemporal_store(val, dst + (int64_t)j * kThreads);
                    }
            return;
        }
        if (fixup) {
            // the parts have been added up into part 0 by split_reduce_kernel; loads go out eight at a time
            const f32x4 *src = (const f32x4 *)prm.split_ws + (int64_t)tail_index * k_split * kTileVecs + wave * 64 + lane;
            constexpr int kVecs = TI * TJ * kVecPerBlk, kBatch = 8;
            static_assert(kVecs % kBatch == 0, "accumulator vectors are loaded in batches of eight");
#pragma unroll
            for (int j0 = 0; j0 < kVecs; j0 += kBatch) {
                f32x4 val[kBatch];
#pragma unroll
                for (int i = 0; i < kBatch; ++i) val[i] = __builtin_nontemporal_load(src + (int64_t)(j0 + i) * kThreads);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < kBatch; ++i) {
                    const int j = j0 + i, blk = j / kVecPerBlk, v = j % kVecPerBlk;
#pragma unroll
                    for (int c = 0; c < 4; ++c) acc[blk / TJ][blk % TJ][4 * v + c] = val[i][c];
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    if constexpr (RAGGED == kRaggedK && QSHAPE == kMC) {
        if (want_bias) {
            // thread t holds CE columns of contraction rows t / Q_CPR (mod kBiasKPI);
            // the kBiasKPI partial sums of a column are added in ascending order
            float *red = (float *)smem;
            __syncthreads();
            // the chunk this thread stages is the one that belongs in its (swizzled) slot
            const int grp = t / Q_CPR, c = (t % Q_CPR) ^ mc_swz<T>(grp);
#pragma unroll
            for (int j = 0; j < CE; ++j) red[grp * BM + c * CE + j] = bsum[j];
            __syncthreads();
            if (t < BM && t < q_valid) {
                float sum = 0.f;
#pragma unroll
                for (int g = 0; g < kBiasKPI; ++g) sum += red[g * BM + t];
                T *dst = (T *)prm.bias_grad + (int64_t)expert * prm.n_rows + mt * BM + t;
                if (prm.accumulate_first && ei == 0) sum += (float)*dst;
                *dst = (T)sum;
            }
        }
    }

    // -- epilogue ------------------------------------------------------------------
    // acc[x][y][4*g + i] is C(row = wave_m0 + MB*y + lb, col = wave_n0 + MB*x + 8*g + 4*hq + i)
    // (32 x 32 blocks: g = 0..3, hq = 0..1; 16 x 16 blocks: g = 0, hq = 0..3): a lane owns
    // runs of 4 consecutive columns in many different rows, which written straight to
    // memory would touch one cache line per row and store.  Instead every wave passes its sub-tile
    // through a private LDS staging area of [WM rows][256 B + 16 B pad] (128 B + 16 B for the
    // 64-column wave tiles of 16-bit types) and moves it between LDS and memory with 16-byte
    // accesses that cover whole row pieces (4 or 8 rows per wave instruction).  Tiles that are read in the epilogue (the saved
    // pre-activation, or C itself when accumulating) come in through the same area.
    if constexpr (RAGGED == kRaggedK && QSHAPE == kMC) {
        if (want_bias) __syncthreads();  // the bias reduction used the start of LDS
    }
    constexpr int kPieceBytes = WN * (int)sizeof(T) < 256 ? WN * (int)sizeof(T) : 256;  // row piece moved per pass
    constexpr int kStgRow = kPieceBytes + 16;    // bytes; the pad spreads rows over the banks
    constexpr int CPP = kPieceBytes / (int)sizeof(T);  // C columns per pass through the staging area
    constexpr int XPP = CPP / MB;                // MFMA block columns per pass
    constexpr int NPASS = WN / CPP;
    unsigned char *stg = smem + (fixup ? 0 : wave) * (WM * kStgRow);
    const T *bias = prm.bias ? (const T *)prm.bias + (int64_t)expert * prm.bias_expert_stride + n0 : nullptr;
    const __amdgpu_buffer_rsrc_t bias_rs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(bias), 0, bias ? p_valid * (int)sizeof(T) : 0, kRsrcFlags);
    T *aux = prm.aux ? (T *)prm.aux + aux_off : nullptr;
    const bool accumulate = (RAGGED == kRaggedK) && prm.accumulate_first && ei == 0;
    constexpr int kPieceChunks = kPieceBytes / 16, kIoRows = 64 / kPieceChunks;
    const int io_r = lane / kPieceChunks, io_c = lane % kPieceChunks;  // coalesced side: kIoRows rows x whole pieces per instruction

    auto lds_sync = [&]() { __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup"); __builtin_amdgcn_wave_barrier(); };

    // The tile in memory is addressed through a buffer resource at its origin (a tile's rows lie
    // within 2 GiB of it): a row or column outside the tile gets an offset past the resource's
    // end, which reads as zero and is dropped on a store -- no branches, so all of a pass's LDS
    // reads (or loads) go out, kIoBatch at a time, before the first of them is waited for.
    constexpr int kIoSteps = WM / kIoRows, kIoBatch = kIoSteps < 8 ? kIoSteps : 8;
    static_assert(kIoSteps % kIoBatch == 0, "row groups of a wave's sub-tile come in whole batches");
    auto tile_offset = [&](int r, int col_base) -> uint32_t {
        return (wave_m0 + r < q_valid && col_base + io_c * CE < p_valid)
                   ? (uint32_t)(((int64_t)(wave_m0 + r) * prm.ldc + col_base + io_c * CE) * (int64_t)sizeof(T))
                   : kOutOfRange;
    };
    // memory -> staging (rows/columns outside the tile read as zero)
    auto stage_in = [&](const T *src, int col_base) {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(src), 0, (int)kOutOfRange, kRsrcFlags);
#pragma unroll
        for (int i0 = 0; i0 < kIoSteps; i0 += kIoBatch) {
            u32x4 v[kIoBatch];
#pragma unroll
            for (int i = 0; i < kIoBatch; ++i)
                v[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)tile_offset((i0 + i) * kIoRows + io_r, col_base), 0, 0);
#pragma unroll
            for (int i = 0; i < kIoBatch; ++i) *(u32x4 *)(stg + ((i0 + i) * kIoRows + io_r) * kStgRow + io_c * 16) = v[i];
        }
    };
    // staging -> memory
    auto stage_out = [&](T *dst, int col_base) {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(dst, 0, (int)kOutOfRange, kRsrcFlags);
#pragma unroll
        for (int i0 = 0; i0 < kIoSteps; i0 += kIoBatch) {
            u32x4 v[kIoBatch];
#pragma unroll
            for (int i = 0; i < kIoBatch; ++i) v[i] = *(const u32x4 *)(stg + ((i0 + i) * kIoRows + io_r) * kStgRow + io_c * 16);
#pragma unroll
            for (int i = 0; i < kIoBatch; ++i)
                __builtin_amdgcn_raw_buffer_store_b128(v[i], rs, (int)tile_offset((i0 + i) * kIoRows + io_r, col_base), 0, 0);
        }
    };
    // accumulator side: 4 consecutive columns of one row
    auto put4 = [&](int row, int col_in_pass, const float (&v)[4]) {
        alignas(16) T res[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) res[i] = (T)v[i];
        unsigned char *p = stg + row * kStgRow + col_in_pass * (int)sizeof(T);
        if (sizeof(T) == 2) *(u32x2 *)p = *(const u32x2 *)res;
        else *(u32x4 *)p = *(const u32x4 *)res;
    };
    auto get4 = [&](int row, int col_in_pass, float (&v)[4]) {
        alignas(16) T in[4];
        const unsigned char *p = stg + row * kStgRow + col_in_pass * (int)sizeof(T);
        if (sizeof(T) == 2) *(u32x2 *)in = *(const u32x2 *)p;
        else *(u32x4 *)in = *(const u32x4 *)p;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (float)in[i];
    };

    // The pre-activation tile that was requested during the last two slabs lies in the slab
    // buffers; every lane takes the 4 values per block it needs into registers (the fragment
    // registers are free now) before the staging area, which overlaps those buffers, is used.
    u32x2 auxv[kAuxPrefetch ? TI : 1][kAuxPrefetch ? TJ : 1];
    if constexpr (kAuxPrefetch) {
        if (aux_pref) {
            // part 0 / 1 went to the P buffers that slabs n-2 / n-1 would have prefetched into,
            // part 2 / 3 to the Q buffers of slabs n-2 / n-1
            const int row_t = wave_m0 + lb;                // tile row of this lane in block row 0
            const int part = row_t >> 6;                   // the same for all block rows of the wave
            const uint32_t part_off = part < 2 ? (uint32_t)(((n_slabs + part) % kPBufs) * P_BYTES)
                                               : (uint32_t)(Q_BASE + ((n_slabs + part) & 1) * Q_BYTES);
#pragma unroll
            for (int x = 0; x < TI; ++x)
#pragma unroll
                for (int y = 0; y < TJ; ++y) {
                    const int rip = (row_t & 63) + y * MB;
                    const int c = ((wave_n0 + x * MB) >> 3) + (hq >> 1);
                    auxv[x][y] = *(const u32x2 *)(smem + part_off + rip * 512 + ((c ^ (rip & 15)) << 4) + (hq & 1) * 8);
                }
            __syncthreads();
        }
    }

    // The activation, the accumulate flag and where the tile that is read comes from are fixed
    // per launch (per tile); the epilogue is instantiated per value so that its element loop is
    // straight-line code.
    auto run_epilogue = [&](auto act_tag, auto accum_tag, auto auxreg_tag) {
    constexpr int ACT = decltype(act_tag)::value;
    constexpr bool kAccum = decltype(accum_tag)::value;
    constexpr bool kAuxRegs = decltype(auxreg_tag)::value;  // the pre-activations are in auxv
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
        const int col_base = wave_n0 + pass * CPP;
        // kind 0: the result; kind 1 (bias+act with a pre-activation buffer): the pre-activation first
        constexpr int kKinds = (EPI == kEpiBiasAct) ? 2 : 1;
#pragma unroll
        for (int kind = kKinds - 1; kind >= 0; --kind) {
            if (EPI == kEpiBiasAct && kind == 1 && !aux) continue;
            constexpr bool reads_tile = (EPI == kEpiDAct) || kAccum;
            if (reads_tile && !kAuxRegs) {
                stage_in(EPI == kEpiDAct ? (const T *)aux : (const T *)Cb, col_base);
                lds_sync();
            }
#pragma unroll
            for (int xx = 0; xx < XPP; ++xx) {
                const int x = pass * XPP + xx;
#pragma unroll
                for (int g = 0; g < kAccRegs / 4; ++g) {
                    const int cip = xx * MB + g * 8 + hq * 4;  // column inside this pass
                    // (columns past the tile, and every column when there is no bias, read as zero)
                    float b4[4];
                    {
                        alignas(16) T bv[4];
                        const int off = (col_base + cip) * (int)sizeof(T);
                        if (sizeof(T) == 2) *(u32x2 *)bv = __builtin_amdgcn_raw_buffer_load_b64(bias_rs, off, 0, 0);
                        else *(u32x4 *)bv = __builtin_amdgcn_raw_buffer_load_b128(bias_rs, off, 0, 0);
#pragma unroll
                        for (int i = 0; i < 4; ++i) b4[i] = (float)bv[i];
                    }
#pragma unroll
                    for (int y = 0; y < TJ; ++y) {
                        const int row = y * MB + lb;
                        float v[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) v[i] = acc[x][y][4 * g + i] + b4[i];
                        if (EPI == kEpiBiasAct && kind == 0) {
#pragma unroll
                            for (int i = 0; i < 4; ++i) v[i] = apply_act<sizeof(T) == 2>(v[i], ACT);
                        }
                        if (reads_tile) {
                            float in[4];
                            if constexpr (kAuxRegs) {
                                alignas(8) T a4[4];
                                *(u32x2 *)a4 = auxv[kAuxPrefetch ? x : 0][kAuxPrefetch ? y : 0];
#pragma unroll
                                for (int i = 0; i < 4; ++i) in[i] = (float)a4[i];
                            } else {
                                get4(row, cip, in);
                            }
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                v[i] = (EPI == kEpiDAct) ? v[i] * act_grad<sizeof(T) == 2>(in[i], ACT) : v[i] + in[i];
                        }
                        put4(row, cip, v);
                    }
                }
            }
            lds_sync();
            stage_out((EPI == kEpiBiasAct && kind == 1) ? aux : Cb, col_base);
            lds_sync();
        }
    }
    };
    typedef std::integral_constant<int, FMOE_ACT_NONE> ActNone;
    auto by_activation = [&](auto auxreg_tag) {
        // (every instantiation is called from one place only, so that it is inlined)
        if constexpr (sizeof(T) == 2) {
            if (prm.activation == kActGeluErf) {
                run_epilogue(std::integral_constant<int, kActGeluErf>{}, std::false_type{}, auxreg_tag);
                return;
            }
        }
        // (a 32-bit type computes GELU with the erf formula anyway)
        if (prm.activation == FMOE_ACT_GELU || prm.activation == kActGeluErf)
            run_epilogue(std::integral_constant<int, FMOE_ACT_GELU>{}, std::false_type{}, auxreg_tag);
        else if (prm.activation == FMOE_ACT_RELU) run_epilogue(std::integral_constant<int, FMOE_ACT_RELU>{}, std::false_type{}, auxreg_tag);
        else run_epilogue(ActNone{}, std::false_type{}, auxreg_tag);
    };
    if constexpr (EPI == kEpiStore) {
        if (accumulate) run_epilogue(ActNone{}, std::true_type{}, std::false_type{});
        else run_epilogue(ActNone{}, std::false_type{}, std::false_type{});
    } else if constexpr (kAuxPrefetch) {
        if (aux_pref) by_activation(std::true_type{});
        else by_activation(std::false_type{});
    } else {
        by_activation(std::false_type{});
    }
#endif  // __HIP_DEVICE_COMPILE__
}

// Adds the k_split partial accumulator tiles of every split tail tile into the first of them,
// in ascending part order (a fixed order: the sum does not depend on scheduling).  One thread
// per 16 bytes of a tile, all of a thread's loads issued before the first add.
template <int kMaxSplit>
__global__ __launch_bounds__(256) void split_reduce_kernel(float *ws, int k_split, int64_t tile_vecs, int64_t total_vecs) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total_vecs) return;
    const int64_t tile = i / tile_vecs, v = i - tile * tile_vecs;
    f32x4 *base = (f32x4 *)ws + tile * k_split * tile_vecs + v;
    f32x4 part[kMaxSplit];
#pragma unroll
    for (int p = 0; p < kMaxSplit; ++p)
        if (p < k_split) part[p] = __builtin_nontemporal_load(base + (int64_t)p * tile_vecs);
    f32x4 sum = part[0];
#pragma unroll
    for (int p = 1; p < kMaxSplit; ++p)
        if (p < k_split) sum += part[p];
    base[0] = sum;
}

// The same for a launch over a device table, sized for the most tail tiles there can be: kPerTile
// workgroups per tile, each adding up its share of the tile in steps of 256 vectors; a workgroup
// works out from the table's tile count whether (and how) the tail was split and leaves at once
// when its tile does not exist.
constexpr int kReducePerTile = 8;
template <int kMaxSplit>
__global__ __launch_bounds__(256) void split_reduce_dev_kernel(float *ws, const int32_t *__restrict__ dev_tab, int tiles_index,
                                                               int tiles_n, int n_slabs, int cus, int slab_weight,
                                                               int64_t tile_vecs) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef const int32_t __attribute__((address_space(4))) *DevTab;
    const int total = ((DevTab)(uintptr_t)dev_tab)[tiles_index] * tiles_n;
    const TailSplit ts = plan_tail_split(total, n_slabs, cus, slab_weight);
    const int tile = blockIdx.x / kReducePerTile, share = blockIdx.x % kReducePerTile;
    if (ts.k_split == 1 || tile >= total - ts.main_tiles) return;
    const int64_t per_share = (tile_vecs + kReducePerTile - 1) / kReducePerTile;
    const int64_t v_end = (share + 1) * per_share < tile_vecs ? (share + 1) * per_share : tile_vecs;
    for (int64_t v = share * per_share + threadIdx.x; v < v_end; v += 256) {
        f32x4 *base = (f32x4 *)ws + (int64_t)tile * ts.k_split * tile_vecs + v;
        f32x4 part[kMaxSplit];
#pragma unroll
        for (int p = 0; p < kMaxSplit; ++p)
            if (p < ts.k_split) part[p] = __builtin_nontemporal_load(base + (int64_t)p * tile_vecs);
        f32x4 sum = part[0];
#pragma unroll
        for (int p = 1; p < kMaxSplit; ++p)
            if (p < ts.k_split) sum += part[p];
        base[0] = sum;
    }
}

// Host-side services of grouped_gemm.hip: compute units of the current device, and a per-stream
// buffer for the partial accumulators of split tail tiles (allocated on first use, kept until
// the process ends; NULL when the allocation fails, in which case nothing is split).
int device_compute_units();
float *split_workspace(hipStream_t stream, size_t bytes);

template <typename T, int BM, int BN, int PS, int QS, int RG, int EPI>
int launch_tiles(GemmParams &prm, hipStream_t stream) {
    constexpr int kWavesM = waves_m_of(BN), kThreads = threads_of(BN);
    // three P and two Q slab buffers, or the epilogue's staging area (one [rows][row piece + 16 B] block per wave)
    constexpr int smem_loop = (3 * BN + 2 * BM) * kSlabBytes;
    constexpr int wave_cols_bytes = BN / kWavesN * (int)sizeof(T);
    constexpr int smem_wave_epi = (BM / kWavesM) * ((wave_cols_bytes < 256 ? wave_cols_bytes : 256) + 16);
    constexpr int smem_epi = kWavesM * kWavesN * smem_wave_epi;
    constexpr int smem = smem_loop > smem_epi ? smem_loop : smem_epi;
    // the opt-in to more than 64 KiB of dynamic LDS is per device (and per kernel instantiation)
    // (0: not tried yet, 1: done, 2: failed -- a failure is reported by every later launch too)
    static std::atomic<int> configured[16];
    auto kern = grouped_gemm_kernel<T, BM, BN, PS, QS, RG, EPI>;
    int dev = 0;
    FMOE_HIP_CHECK(hipGetDevice(&dev));
    FMOE_REQUIRE(dev >= 0 && dev < 16, "device index %d out of range", dev);
    if (configured[dev].load(std::memory_order_acquire) != 1) {
        // (two threads may both make the call; it is idempotent)
        const hipError_t attr_err = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        configured[dev].store(attr_err == hipSuccess ? 1 : 2, std::memory_order_release);
        FMOE_HIP_CHECK(attr_err);
    }
    if (prm.total_tiles <= 0) return FMOE_OK;
    prm.main_tiles = prm.total_tiles;
    prm.k_split = 1;
    prm.split_slabs = 0;
    prm.fixup = 0;
    prm.split_ws = nullptr;
    int64_t grid64;
    if (RG == kRaggedRows) {
        constexpr int BKE = kSlabBytes / (int)sizeof(T);
        const int n_slabs = (prm.k_extent + BKE - 1) / BKE;
        constexpr int kWeight = slab_weight_of<T>();
        if (prm.dev_tab != nullptr) {
            // the host does not know the tile count: with a workspace from the caller, every workgroup plans the
            // split itself, and the launch is sized for the most parts there can be (one per compute unit)
            prm.dev_cus = 0;
            if (prm.dev_split_ws != nullptr && tail_split_possible(n_slabs, kWeight)) {
                prm.dev_cus = device_compute_units();
                prm.split_ws = prm.dev_split_ws;
            }
            grid64 = ((int64_t)prm.total_tiles + 7) / 8 * 8 + prm.dev_cus;
        } else {
            const TailSplit ts = plan_tail_split(prm.total_tiles, n_slabs, device_compute_units(), kWeight);
            if (ts.k_split > 1) {
                const int tail = prm.total_tiles - ts.main_tiles;
                float *ws = split_workspace(stream, (size_t)tail * ts.k_split * BM * BN * sizeof(float));
                if (ws != nullptr) {
                    prm.split_ws = ws;
                    prm.main_tiles = ts.main_tiles;
                    prm.k_split = ts.k_split;
                    prm.split_slabs = ts.split_slabs;
                }
            }
            // whole tiles rounded up to a multiple of 8 (one range per XCD), then the parts of the tail tiles
            grid64 = ((int64_t)prm.main_tiles + 7) / 8 * 8 + (int64_t)(prm.total_tiles - prm.main_tiles) * prm.k_split;
        }
    } else {
        // 8 XCDs x experts x an eighth (rounded up) of one expert's tiles -- the kernel drops the surplus workgroups
        grid64 = (int64_t)8 * prm.tab.n * (((int64_t)prm.tiles_m * prm.tiles_n + 7) / 8);
    }
    if (grid64 > (int64_t)INT32_MAX) return fail(FMOE_ELIMIT, "grouped GEMM: grid of %lld workgroups", (long long)grid64);
    const int grid = (int)grid64;
    ProfileScope prof(prm.profile_class, prm.profile_work, stream);
    kern<<<grid, kThreads, smem, stream>>>(prm);
    FMOE_LAUNCH_CHECK();
    if (prm.k_split > 1) {
        // the parts are complete when the first launch has ended: add them up, then run the epilogue,
        // one wave (its share of the tile) per workgroup
        const int tail = prm.total_tiles - prm.main_tiles;
        const int64_t tile_vecs = (int64_t)BM * BN / 4, total_vecs = tile_vecs * tail;
        split_reduce_kernel<kMaxSplit><<<(unsigned)((total_vecs + 255) / 256), 256, 0, stream>>>(prm.split_ws, prm.k_split, tile_vecs, total_vecs);
        FMOE_LAUNCH_CHECK();
        prm.fixup = 1;
        kern<<<(prm.total_tiles - prm.main_tiles) * kWavesM * kWavesN, 64, smem_wave_epi, stream>>>(prm);
        FMOE_LAUNCH_CHECK();
        prm.fixup = 0;
    } else if (RG == kRaggedRows && prm.dev_tab != nullptr && prm.dev_cus > 0) {
        // device table: the same two steps, sized for the most tail tiles a split can have (half the chip)
        constexpr int BKE = kSlabBytes / (int)sizeof(T);
        const int max_tail = prm.dev_cus / 2;
        const int64_t tile_vecs = (int64_t)BM * BN / 4;
        split_reduce_dev_kernel<kMaxSplit><<<(unsigned)(max_tail * kReducePerTile), 256, 0, stream>>>(
            prm.split_ws, prm.dev_tab, BM == 256 ? segtab::kTiles256 : segtab::kTiles128, prm.tiles_n,
            (prm.k_extent + BKE - 1) / BKE, prm.dev_cus, slab_weight_of<T>(), tile_vecs);
        FMOE_LAUNCH_CHECK();
        prm.fixup = 1;
        kern<<<max_tail * kWavesM * kWavesN, 64, smem_wave_epi, stream>>>(prm);
        FMOE_LAUNCH_CHECK();
        prm.fixup = 0;
    }
    return FMOE_OK;
}

// Tile counts, then the launch for the requested epilogue.  prm.block_m x prm.block_n (256 x 256,
// 128 x 256 or 128 x 128, chosen by the host from the segment lengths) is the tile.
// EPI_MASK lists the epilogues a product can be asked for, so that only those kernels
// are built.
template <typename T, int BM, int BN, int PS, int QS, int RG, int EPI_MASK>
int launch_for_height(GemmParams &prm, int epi, hipStream_t stream) {
    prm.tiles_n = (int)ceil_div(prm.n_cols, BN);
    int64_t total;
    if (RG == kRaggedRows) {
        prm.tiles_m = 0;
        // device table: the most row tiles its rows can make (the kernel drops the surplus workgroups)
        total = (prm.dev_tab ? segtab::cap_tiles(prm.dev_rows_cap, prm.tab.n, BM) : (int64_t)prm.tab.tile[prm.tab.n]) * prm.tiles_n;
        if (prm.dev_tab)
            prm.dev_map_off = (int32_t)(BM == 256 ? segtab::map256_off(prm.tab.n) : segtab::map128_off(prm.dev_rows_cap, prm.tab.n));
    } else {
        prm.tiles_m = (int)ceil_div(prm.n_rows, BM);
        total = (int64_t)prm.tab.n * prm.tiles_m * prm.tiles_n;
    }
    if (total > (int64_t)INT32_MAX - 8) return fail(FMOE_ELIMIT, "grouped GEMM: %lld tiles exceed the grid limit", (long long)total);
    prm.total_tiles = (int)total;
    if constexpr ((EPI_MASK >> kEpiStore) & 1)
        if (epi == kEpiStore) return launch_tiles<T, BM, BN, PS, QS, RG, kEpiStore>(prm, stream);
    if constexpr ((EPI_MASK >> kEpiBiasAct) & 1)
        if (epi == kEpiBiasAct) return launch_tiles<T, BM, BN, PS, QS, RG, kEpiBiasAct>(prm, stream);
    if constexpr ((EPI_MASK >> kEpiDAct) & 1)
        if (epi == kEpiDAct) return launch_tiles<T, BM, BN, PS, QS, RG, kEpiDAct>(prm, stream);
    return fail(FMOE_EINVAL, "epilogue %d is not built for this product", epi);
}

template <typename T, int PS, int QS, int RG, int EPI_MASK>
int launch_by_epilogue(GemmParams &prm, int epi, hipStream_t stream) {
    if (prm.block_m == 128 && prm.block_n == 128) return launch_for_height<T, 128, 128, PS, QS, RG, EPI_MASK>(prm, epi, stream);
    if (prm.block_m == 128 && prm.block_n == 256) return launch_for_height<T, 128, 256, PS, QS, RG, EPI_MASK>(prm, epi, stream);
    if (prm.block_m == 256 && prm.block_n == 256) return launch_for_height<T, 256, 256, PS, QS, RG, EPI_MASK>(prm, epi, stream);
    return fail(FMOE_EINVAL, "tile %d x %d is not built", prm.block_m, prm.block_n);
}

}  // namespace gemm

// Defined in gemm_inst.hip, once per (element type, product).
#define FMOE_DECLARE_MFMA(NAME) int NAME(gemm::GemmParams &prm, int epilogue, hipStream_t stream)
FMOE_DECLARE_MFMA(launch_mfma_bf16_fwd);
FMOE_DECLARE_MFMA(launch_mfma_bf16_dgrad);
FMOE_DECLARE_MFMA(launch_mfma_bf16_wgrad);
FMOE_DECLARE_MFMA(launch_mfma_f16_fwd);
FMOE_DECLARE_MFMA(launch_mfma_f16_dgrad);
FMOE_DECLARE_MFMA(launch_mfma_f16_wgrad);
FMOE_DECLARE_MFMA(launch_mfma_f32_fwd);
FMOE_DECLARE_MFMA(launch_mfma_f32_dgrad);
FMOE_DECLARE_MFMA(launch_mfma_f32_wgrad);
// double precision, and any type with feature sizes or pointers off the 16-byte grid; all three products
// (0 forward, 1 data gradient, 2 weight gradient): gemm_any.hip
int launch_mfma_any(gemm::GemmParams &prm, int dtype, int product, int epilogue, hipStream_t stream);

}  // namespace fmoe
