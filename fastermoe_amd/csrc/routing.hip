// Routing bookkeeping and capacity balancing for gfx950.
//
// Every entry point that has to order slots ("which slots of expert e come
// first") is built on one primitive: the RANK of a slot among the slots of the
// same expert with a lower flat index.  The rank is computed without atomics on
// shared counters, so results do not depend on scheduling:
//
//   1. hist   : each 256-thread workgroup owns kSlotsPerBlock consecutive slots
//               and writes its per-expert histogram (LDS-staged) to scratch;
//   2. scan   : per expert, an exclusive prefix over the workgroups (and, for
//               fmoe_route, the cumsum over experts);
//   3. apply  : each wave walks its 512 slots in order; inside a 64-slot step
//               the rank comes from a ballot-built match mask and a popcount of
//               the lower lanes, across steps from a wave-private LDS counter.
//
// The index arrays are a few hundred KB at most, so these kernels are bound by
// launch and memory latency, not by HBM bandwidth; the design keeps them to
// three short launches with coalesced 8-byte loads.
#include "common.hpp"

#include <mutex>
#include <type_traits>

namespace fmoe {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kStepsPerWave = 8;
constexpr int kSlotsPerWave = kWave * kStepsPerWave;          // 512
constexpr int kSlotsPerBlock = kSlotsPerWave * kWavesPerBlock; // 2048
constexpr int64_t kMaxExpert = 8192;  // 4 wave-private int32 tables in 160 KB LDS

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

__device__ __forceinline__ uint64_t lanes_below() {
    return (1ull << lane_id()) - 1ull;
}

// Mask of the lanes of this wave that hold the same key; lanes with
// valid == false get 0.  nbits = number of significant key bits.
__device__ __forceinline__ uint64_t match_mask(int key, bool valid, int nbits) {
    uint64_t peers = __ballot(valid);
    for (int b = 0; b < nbits; ++b) {
        const bool bit = (key >> b) & 1;
        const uint64_t vote = __ballot(valid && bit);
        peers &= bit ? vote : ~vote;
    }
    return valid ? peers : 0ull;
}

// Orders this wave's LDS accesses: the lanes of a wave run in lock-step and the LDS serves a
// wave's instructions in order, so a wave-private table needs no workgroup barrier -- only
// the compiler must keep the accesses in program order.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Adds this wave's 64 keys to its private table without atomics: of the lanes that hold the
// same key, the lowest one adds their number.
__device__ __forceinline__ void wave_bins_add(int32_t *mine, int key, bool valid, uint64_t peers) {
    if (valid && (peers & lanes_below()) == 0) mine[key] += __popcll(peers);
    wave_lds_sync();
}

// ---------------------------------------------------------------- count ----

// Wave-private LDS histograms filled without atomics, then one global integer add per
// workgroup and non-empty bin (the entry point ADDS to the caller's counts, as the
// reference kernel does; integer adds commute, so the result does not depend on scheduling).
__global__ __launch_bounds__(kBlock) void expert_count_kernel(
    const int64_t *__restrict__ gate, int32_t *__restrict__ count,
    int64_t n_slots, int n_expert, int nbits) {
    extern __shared__ int32_t bins[];  // [kWavesPerBlock][n_expert]
    int32_t *mine = bins + (threadIdx.x / kWave) * n_expert;
    for (int e = threadIdx.x; e < kWavesPerBlock * n_expert; e += kBlock) bins[e] = 0;
    __syncthreads();
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    const int64_t rounds = (n_slots + stride - 1) / stride;  // the same for every lane: ballots need whole waves
    for (int64_t r = 0; r < rounds; ++r) {
        const int64_t i = r * stride + (int64_t)blockIdx.x * kBlock + threadIdx.x;
        int64_t g = -1;
        if (i < n_slots) g = gate[i];
        const bool valid = g >= 0 && g < n_expert;
        const int key = valid ? (int)g : 0;
        wave_bins_add(mine, key, valid, match_mask(key, valid, nbits));
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n_expert; e += kBlock) {
        int32_t c = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) c += bins[w * n_expert + e];
        if (c) atomicAdd(&count[e], c);
    }
}

// ----------------------------------------------------------------- hist ----

// block_hist[b][e] = #slots of expert e in workgroup b's slot range; wave-private tables
// filled without atomics, added up at the end.
__global__ __launch_bounds__(kBlock) void block_hist_kernel(
    const int64_t *__restrict__ gate, int32_t *__restrict__ block_hist,
    int64_t n_slots, int n_expert, int nbits) {
    extern __shared__ int32_t bins[];  // [kWavesPerBlock][n_expert]
    const int wave = threadIdx.x / kWave;
    int32_t *mine = bins + wave * n_expert;
    for (int e = threadIdx.x; e < kWavesPerBlock * n_expert; e += kBlock) bins[e] = 0;
    __syncthreads();
    const int64_t wave_base = (int64_t)blockIdx.x * kSlotsPerBlock + (int64_t)wave * kSlotsPerWave;
#pragma unroll
    for (int s = 0; s < kStepsPerWave; ++s) {
        const int64_t i = wave_base + s * kWave + lane_id();
        int64_t g = -1;
        if (i < n_slots) g = gate[i];
        const bool valid = g >= 0 && g < n_expert;
        const int key = valid ? (int)g : 0;
        wave_bins_add(mine, key, valid, match_mask(key, valid, nbits));
    }
    __syncthreads();
    int32_t *dst = block_hist + (int64_t)blockIdx.x * n_expert;
    for (int e = threadIdx.x; e < n_expert; e += kBlock) {
        int32_t c = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) c += bins[w * n_expert + e];
        dst[e] = c;
    }
}

// ----------------------------------------------------------------- scan ----

enum ScanMode { kScanAssign = 0, kScanPrune = 1 };

// One thread per expert: block_hist[.][e] -> exclusive prefix over workgroups
// (in place).  limit[e] is the caller's per-expert int32 array (cum_count for
// assign_pos, remaining capacity for prune); its old value is parked in
// limit_old[e] for the apply kernel and the array is updated the way the
// reference kernel leaves it (every slot subtracts one).
__global__ __launch_bounds__(kBlock) void block_scan_kernel(
    int32_t *__restrict__ block_hist, int n_blocks, int n_expert,
    int32_t *__restrict__ limit, int32_t *__restrict__ limit_old) {
    const int e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_expert) return;
    int32_t run = 0;
    for (int b = 0; b < n_blocks; ++b) {
        int32_t *cell = block_hist + (int64_t)b * n_expert + e;
        const int32_t c = *cell;
        *cell = run;
        run += c;
    }
    const int32_t old = limit[e];
    limit_old[e] = old;
    limit[e] = old - run;
}

// fmoe_route: a single 1024-thread workgroup does the per-expert prefix over
// workgroups and then the inclusive cumsum over experts.
constexpr int kRouteScanBlock = 1024;
__global__ __launch_bounds__(kRouteScanBlock) void route_scan_kernel(
    int32_t *__restrict__ block_hist, int n_blocks, int n_expert,
    int64_t *__restrict__ expert_count, int32_t *__restrict__ cum_incl) {
    __shared__ int32_t wave_sum[kRouteScanBlock / kWave];
    __shared__ int32_t carry_s;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    for (int e0 = 0; e0 < n_expert; e0 += kRouteScanBlock) {
        const int e = e0 + threadIdx.x;
        int32_t run = 0;
        if (e < n_expert) {
            for (int b = 0; b < n_blocks; ++b) {
                int32_t *cell = block_hist + (int64_t)b * n_expert + e;
                const int32_t c = *cell;
                *cell = run;
                run += c;
            }
            expert_count[e] = run;
        }
        // inclusive scan of `run` over the workgroup
        int32_t v = run;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const int32_t up = __shfl_up(v, off, kWave);
            if (lane_id() >= off) v += up;
        }
        const int wave = threadIdx.x / kWave;
        if (lane_id() == kWave - 1) wave_sum[wave] = v;
        __syncthreads();
        int32_t before = carry_s;
        for (int w = 0; w < wave; ++w) before += wave_sum[w];
        if (e < n_expert) cum_incl[e] = v + before;
        __syncthreads();
        if (threadIdx.x == kRouteScanBlock - 1) carry_s = v + before;
        __syncthreads();
    }
}

// ---------------------------------------------------------------- apply ----

enum ApplyMode { kApplyAssign = 0, kApplyPrune = 1 };

// Recomputes the per-wave histograms of this workgroup's slots, turns them into
// per-wave starting ranks (block prefix from the scan + waves before this one)
// and walks the slots in order.
//   assign: pos[limit_old[e] - 1 - rank] = slot   (+ slot_to_row[slot] = that); pos[i] = -1 for i >= limit_old[E-1]
//   prune : out[slot] = rank < limit_old[e] ? e : -1
template <int MODE>
__global__ __launch_bounds__(kBlock) void rank_apply_kernel(
    const int64_t *__restrict__ gate, const int32_t *__restrict__ block_base,
    const int32_t *__restrict__ limit_old, int64_t *__restrict__ out,
    int64_t *__restrict__ slot_to_row, int64_t n_slots, int64_t n_out, int n_expert, int nbits, int fill_tail) {
    extern __shared__ int32_t lds[];  // [kWavesPerBlock][n_expert]
    const int wave = threadIdx.x / kWave;
    int32_t *mine = lds + wave * n_expert;
    for (int e = threadIdx.x; e < kWavesPerBlock * n_expert; e += kBlock) lds[e] = 0;
    __syncthreads();

    const int64_t wave_base = (int64_t)blockIdx.x * kSlotsPerBlock + (int64_t)wave * kSlotsPerWave;
    int keys[kStepsPerWave];
    uint64_t peers[kStepsPerWave];
#pragma unroll
    for (int s = 0; s < kStepsPerWave; ++s) {
        const int64_t i = wave_base + s * kWave + lane_id();
        int64_t g = -1;
        if (i < n_slots) g = gate[i];
        keys[s] = (g >= 0 && g < n_expert) ? (int)g : -1;
        peers[s] = match_mask(keys[s], keys[s] >= 0, nbits);
        wave_bins_add(mine, keys[s], keys[s] >= 0, peers[s]);
    }
    __syncthreads();
    // per-wave histogram -> starting rank of this wave for every expert
    const int32_t *bb = block_base + (int64_t)blockIdx.x * n_expert;
    for (int e = threadIdx.x; e < n_expert; e += kBlock) {
        int32_t run = bb[e];
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) {
            const int32_t c = lds[w * n_expert + e];
            lds[w * n_expert + e] = run;
            run += c;
        }
    }
    __syncthreads();

    // from here on a wave only touches its own table: wave-level ordering is enough
#pragma unroll
    for (int s = 0; s < kStepsPerWave; ++s) {
        const int64_t i = wave_base + s * kWave + lane_id();
        const int key = keys[s];
        const bool valid = key >= 0;
        int32_t rank = 0;
        if (valid) rank = mine[key] + __popcll(peers[s] & lanes_below());
        wave_lds_sync();  // every lane has read its counter before the leaders bump it
        wave_bins_add(mine, key, valid, peers[s]);
        if (MODE == kApplyAssign) {
            if (valid) {
                const int64_t row = (int64_t)limit_old[key] - 1 - rank;
                if (row >= 0 && row < n_out) out[row] = i;  // a short pos buffer is never overrun
                if (slot_to_row) slot_to_row[i] = row;
            } else if (slot_to_row && i < n_slots) {
                slot_to_row[i] = -1;
            }
            // the entries of `out` past the last routed slot name no slot: -1, so that a row gather over
            // the whole buffer can be launched before the host knows how many slots were routed
            // (fill_tail: limit_old is this library's own inclusive count prefix, so its last entry is the total)
            if (fill_tail && i < n_slots && i < n_out && i >= (int64_t)limit_old[n_expert - 1]) out[i] = -1;
        } else {
            if (i < n_slots) out[i] = (valid && rank < limit_old[key]) ? (int64_t)key : -1;
        }
    }
}

// ----------------------------------------------------------------- gate ----

// Keeps the K largest (value, expert) pairs seen so far in descending order of the value.  A
// later value only displaces a strictly smaller one, so ties go to the lower expert index; a
// place that is still empty (idx < 0) takes anything, so a row with fewer than K values above
// -inf still names K experts (torch.topk, which this stands in for, does too; unlike torch.topk,
// which ranks NaN above everything, a NaN is taken as -inf here).
template <int K>
__device__ __forceinline__ void topk_insert(float (&val)[K], int (&idx)[K], float x, int e) {
    x = x != x ? -__builtin_inff() : x;   // a NaN ranks (and scores) as -inf
#pragma unroll
    for (int j = K - 1; j >= 0; --j) {
        const int up = j > 0 ? j - 1 : 0;
        const bool here = x > val[j] || idx[j] < 0;                   // x belongs at or above place j
        const bool above = j > 0 && (x > val[up] || idx[up] < 0);      // ... above it: place j takes its upper neighbour
        val[j] = here ? (above ? val[up] : x) : val[j];
        idx[j] = here ? (above ? idx[up] : e) : idx[j];
    }
}

// Top-k of the gate logits, the scores of the selected experts and the per-workgroup expert
// histogram that the routing scan starts from, in one pass over the logits.
//
// A workgroup owns kSlotsPerBlock consecutive (token, choice) slots -- the same slots as
// workgroup b of rank_apply_kernel -- i.e. kSlotsPerBlock / K tokens, 8 / K per thread.  A lane
// reads its token's row of logits (16 bytes at a time when the rows are aligned) and keeps the K
// largest in a sorted register list: an insertion is K compare-selects, there is no traffic
// between lanes, and a later logit only displaces a strictly smaller one, so ties go to the
// lower expert index.  The choices come out in descending order of the logit.  The wave then
// adds the selected experts to its private table, one 64-key step per choice.
// score_mode 0: the selected logit itself; 1: softmax over the K selected logits.
template <typename T, int K>
__global__ __launch_bounds__(kBlock) void gate_topk_hist_kernel(
    const T *__restrict__ logits, int64_t n_tokens, int n_expert, int score_mode, int vector_rows,
    int64_t *__restrict__ topk_idx, T *__restrict__ topk_score, int32_t *__restrict__ block_hist, int nbits) {
    extern __shared__ int32_t bins[];  // [kWavesPerBlock][n_expert]
    int32_t *mine = bins + (threadIdx.x / kWave) * n_expert;
    for (int e = threadIdx.x; e < kWavesPerBlock * n_expert; e += kBlock) bins[e] = 0;
    __syncthreads();

    constexpr int kTokensPerBlock = kSlotsPerBlock / K, kTokensPerThread = kTokensPerBlock / kBlock;
    constexpr int kVec = 16 / (int)sizeof(T);
    const float kLowest = -__builtin_inff();
    for (int it = 0; it < kTokensPerThread; ++it) {
        const int64_t token = (int64_t)blockIdx.x * kTokensPerBlock + it * kBlock + threadIdx.x;
        const bool live = token < n_tokens;
        float val[K];
        int idx[K];
#pragma unroll
        for (int j = 0; j < K; ++j) { val[j] = kLowest; idx[j] = -1; }
        auto insert = [&](float x, int e) { topk_insert<K>(val, idx, x, e); };
        if (live) {
            const T *row = logits + token * n_expert;
            int e = 0;
            if (vector_rows) {
                for (; e + kVec <= n_expert; e += kVec) {
                    alignas(16) T chunk[kVec];
                    *(uint4 *)chunk = *(const uint4 *)(row + e);
#pragma unroll
                    for (int c = 0; c < kVec; ++c) insert((float)chunk[c], e + c);
                }
            }
            for (; e < n_expert; ++e) insert((float)row[e], e);
        }
        float score[K];
#pragma unroll
        for (int j = 0; j < K; ++j) score[j] = val[j];
        if (score_mode == 1) {
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < K; ++j) { score[j] = idx[j] >= 0 ? __expf(val[j] - val[0]) : 0.f; sum += score[j]; }
#pragma unroll
            for (int j = 0; j < K; ++j) score[j] /= sum;
        }
#pragma unroll
        for (int j = 0; j < K; ++j) {
            const bool chosen = live && idx[j] >= 0;
            if (live) {
                topk_idx[token * K + j] = idx[j];
                topk_score[token * K + j] = (T)(chosen ? score[j] : 0.f);
            }
            wave_bins_add(mine, chosen ? idx[j] : 0, chosen, match_mask(chosen ? idx[j] : 0, chosen, nbits));
        }
    }
    __syncthreads();
    int32_t *dst = block_hist + (int64_t)blockIdx.x * n_expert;
    for (int e = threadIdx.x; e < n_expert; e += kBlock) {
        int32_t c = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) c += bins[w * n_expert + e];
        dst[e] = c;
    }
}

// The gate's linear layer, its top-k and the scores in one kernel, for up to 64 experts: the logits
// x W^T + b (fmoe/gates/naive_gate.py:26-31) are formed in registers and LDS and never written
// to memory.  A workgroup owns kGateTokens tokens; its four waves split the contraction (wave w
// takes the steps w, w + 4, ... of 128 bytes per row) and feed the MFMA straight from global
// memory -- for the 16 x 16 block shapes a lane's operand is 16 contiguous bytes of one row of W
// (expert lb of a 16-expert block) or of x (token lb of a 16-token block), so there is no staging
// -- then leave their partial [expert][token] tiles in LDS.  Thread t < kGateTokens adds the four
// partials of its token's logits in wave order (a fixed order), adds the bias, rounds to the
// element type (what the layer's own output would have been) and keeps the K largest exactly as
// gate_topk_hist_kernel does.  The routing histogram is left to the routing kernels that follow:
// the contraction wants many small workgroups, the histogram few large ones.
constexpr int kGateTokens = 32, kGateMaxExpert = 64, kGateStride = kGateTokens + 4;

template <typename T, int K, int kEB>
__global__ __launch_bounds__(kBlock) void gate_linear_topk_kernel(
    const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ bias, int64_t n_tokens, int d,
    int n_expert, int score_mode, int64_t *__restrict__ topk_idx, T *__restrict__ topk_score) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    extern __shared__ float part_lds[];   // [kWavesPerBlock][16 n_eb][kGateStride]
    constexpr int kTB = kGateTokens / 16;   // kEB: 16-expert blocks this instantiation holds accumulators for
    constexpr int kPer = 16 / (int)sizeof(T);       // elements per 16-byte operand
    constexpr int kStep = 8 * kPer;                 // contraction elements per step of a wave (128 bytes per row)
    const int lane = lane_id(), wave = threadIdx.x / kWave, lb = lane & 15, hq = lane >> 4;
    const int64_t token0 = (int64_t)blockIdx.x * kGateTokens;
    const int n_eb = (n_expert + 15) / 16;

    f32x4 acc[kEB][kTB];
#pragma unroll
    for (int eb = 0; eb < kEB; ++eb)
#pragma unroll
        for (int tb = 0; tb < kTB; ++tb) acc[eb][tb] = f32x4{0.f, 0.f, 0.f, 0.f};
    const T *wrow[kEB];
    const T *xrow[kTB];
    bool wok[kEB], xok[kTB];
#pragma unroll
    for (int eb = 0; eb < kEB; ++eb) {
        wok[eb] = eb * 16 + lb < n_expert;
        wrow[eb] = w + (int64_t)(wok[eb] ? eb * 16 + lb : 0) * d;
    }
#pragma unroll
    for (int tb = 0; tb < kTB; ++tb) {
        xok[tb] = token0 + tb * 16 + lb < n_tokens;
        xrow[tb] = x + (xok[tb] ? token0 + tb * 16 + lb : 0) * d;
    }
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 zero4 = {0, 0, 0, 0};
    auto mma = [&](const u32x4 (&a)[kEB], const u32x4 (&b)[kTB]) {
#pragma unroll
        for (int eb = 0; eb < kEB; ++eb) {
            if (eb >= n_eb) continue;
#pragma unroll
            for (int tb = 0; tb < kTB; ++tb) {
                if constexpr (sizeof(T) == 4) {
                    const float *af = (const float *)&a[eb], *bf = (const float *)&b[tb];
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[eb][tb] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[j], bf[j], acc[eb][tb], 0, 0, 0);
                } else if constexpr (std::is_same<T, __bf16>::value) {
                    acc[eb][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[eb]), __builtin_bit_cast(bf16x8, b[tb]), acc[eb][tb], 0, 0, 0);
                } else {
                    acc[eb][tb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a[eb]), __builtin_bit_cast(f16x8, b[tb]), acc[eb][tb], 0, 0, 0);
                }
            }
        }
    };
    // rows outside the problem read row 0 (and are dropped at the end): no bounds checks on the way.
    // A wave's step covers 128 bytes of every row -- whole cache lines, as two 64-byte halves (the
    // operands of two products) -- and the four waves take the steps in turn.
    constexpr int kUnroll = 2, kStride = kWavesPerBlock * kStep;
    // Workgroups start at different places of the contraction and wrap around: in step with each
    // other they would all ask for the same columns of their rows at the same time, which lie a whole
    // row length apart and so fall on a few memory channels.  (The order of the fp32 additions
    // then depends on where in the batch a token stands; the result stays a fixed function of the input.)
    const int n_groups = (d + kUnroll * kStride - 1) / (kUnroll * kStride);
    const int first = (int)((blockIdx.x * 7u) % (unsigned)n_groups);
    for (int gi = 0; gi < n_groups; ++gi) {
        const int g = gi + first < n_groups ? gi + first : gi + first - n_groups;
        const int k0 = g * (kUnroll * kStride) + wave * kStep;
        if (k0 + (kUnroll - 1) * kStride + kStep <= d) {
            // a whole group of kUnroll steps: every load goes out before the first product needs one
            u32x4 a[kUnroll][2][kEB], b[kUnroll][2][kTB];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const int k = k0 + u * kStride + (c * 4 + hq) * kPer;
#pragma unroll
                    for (int tb = 0; tb < kTB; ++tb) b[u][c][tb] = *(const u32x4 *)(xrow[tb] + k);
#pragma unroll
                    for (int eb = 0; eb < kEB; ++eb) a[u][c][eb] = eb < n_eb ? *(const u32x4 *)(wrow[eb] + k) : zero4;
                }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
#pragma unroll
                for (int c = 0; c < 2; ++c) mma(a[u][c], b[u][c]);
        } else {
            for (int ks = k0; ks < d && ks < k0 + kUnroll * kStride; ks += kStride) {
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const int k = ks + (c * 4 + hq) * kPer;   // d is a multiple of kPer: a chunk lies inside the row or outside it
                    u32x4 a[kEB], b[kTB];
#pragma unroll
                    for (int tb = 0; tb < kTB; ++tb) b[tb] = k < d ? *(const u32x4 *)(xrow[tb] + k) : zero4;
#pragma unroll
                    for (int eb = 0; eb < kEB; ++eb) a[eb] = (eb < n_eb && k < d) ? *(const u32x4 *)(wrow[eb] + k) : zero4;
                    mma(a, b);
                }
            }
        }
    }
    // lane (lb, hq) holds, per block pair, experts 4 hq .. 4 hq + 3 of the expert block for token lb of the token block
#pragma unroll
    for (int eb = 0; eb < kEB; ++eb)
#pragma unroll
        for (int tb = 0; tb < kTB; ++tb)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (eb < n_eb) part_lds[((wave * n_eb + eb) * 16 + 4 * hq + r) * kGateStride + tb * 16 + lb] = acc[eb][tb][r];
    __syncthreads();

    const int t = threadIdx.x;
    const int64_t token = token0 + t;
    if (t >= kGateTokens || token >= n_tokens) return;
    float val[K];
    int idx[K];
#pragma unroll
    for (int j = 0; j < K; ++j) { val[j] = -__builtin_inff(); idx[j] = -1; }
    for (int e = 0; e < n_expert; ++e) {
        const float *p = part_lds + e * kGateStride + t;
        const int ws = n_eb * 16 * kGateStride;   // one wave's tile
        float logit = ((p[0] + p[ws]) + p[2 * ws]) + p[3 * ws];
        if (bias != nullptr) logit += (float)bias[e];
        topk_insert<K>(val, idx, (float)(T)logit, e);
    }
    float score[K];
#pragma unroll
    for (int j = 0; j < K; ++j) score[j] = val[j];
    if (score_mode == 1) {
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < K; ++j) { score[j] = idx[j] >= 0 ? __expf(val[j] - val[0]) : 0.f; sum += score[j]; }
#pragma unroll
        for (int j = 0; j < K; ++j) score[j] /= sum;
    }
#pragma unroll
    for (int j = 0; j < K; ++j) {
        topk_idx[token * K + j] = idx[j];
        topk_score[token * K + j] = (T)(idx[j] >= 0 ? score[j] : 0.f);
    }
}

// ----------------------------------------------------------- noisy gate ----

// Noisy top-k gating (Shazeer et al. 2017, sec. 2.1 and appendix A; fmoe/gates/noisy_gate.py:113-144)
// in training mode, one pass over the two logit matrices and the noise:
//   std_e   = softplus(raw_e) + eps            noisy_e = clean_e + noise_e * std_e
//   v_0 >= ... >= v_K : the K + 1 largest noisy logits (ties to the lower expert), experts i_0 .. i_K
//   gates_j = softmax(v_0 .. v_{K-1})_j
//   P_e     = Phi((clean_e - (noisy_e > v_K ? v_K : v_{K-1})) / std_e)      load_e = sum over tokens of P_e
// A workgroup owns the same kSlotsPerBlock / K tokens as in gate_topk_hist_kernel and leaves the
// routing histogram of its selections for route_scan_kernel.  The load is summed without atomics:
// a wave adds its 64 tokens' P_e by a butterfly of lane exchanges, wave-private LDS tables take
// the sums, the four tables are added in wave order and written per workgroup; the caller adds
// the workgroups' rows.  thr_val / thr_idx keep (v_{K-1}, v_K) and (i_{K-1}, i_K) for the backward.
__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(__expf(x)); }
__device__ __forceinline__ float normal_cdf_f(float z) { return 0.5f * (1.f + erff(z * 0.70710678118654752440f)); }

template <typename T, int K>
__global__ __launch_bounds__(kBlock) void noisy_gate_forward_kernel(
    const T *__restrict__ clean, const T *__restrict__ raw, const T *__restrict__ noise, float eps, int64_t n_tokens,
    int n_expert, int64_t *__restrict__ topk_idx, T *__restrict__ gates, float *__restrict__ thr_val,
    int32_t *__restrict__ thr_idx, float *__restrict__ load_partial, int32_t *__restrict__ block_hist, int nbits) {
    extern __shared__ int32_t bins[];  // [kWavesPerBlock][n_expert] int32 histogram, then the same of float load sums
    const int wave = threadIdx.x / kWave;
    int32_t *mine = bins + wave * n_expert;
    float *loads = (float *)(bins + kWavesPerBlock * n_expert);
    float *my_load = loads + wave * n_expert;
    for (int e = threadIdx.x; e < kWavesPerBlock * n_expert; e += kBlock) { bins[e] = 0; loads[e] = 0.f; }
    __syncthreads();

    constexpr int kTokensPerBlock = kSlotsPerBlock / K, kTokensPerThread = kTokensPerBlock / kBlock;
    for (int it = 0; it < kTokensPerThread; ++it) {
        const int64_t token = (int64_t)blockIdx.x * kTokensPerBlock + it * kBlock + threadIdx.x;
        const bool live = token < n_tokens;
        const int64_t row = (live ? token : 0) * n_expert;
        float val[K + 1];
        int idx[K + 1];
#pragma unroll
        for (int j = 0; j <= K; ++j) { val[j] = -__builtin_inff(); idx[j] = -1; }
        for (int e = 0; e < n_expert; ++e) {
            const float std_e = softplus_f((float)raw[row + e]) + eps;
            topk_insert<K + 1>(val, idx, (float)clean[row + e] + (float)noise[row + e] * std_e, e);
        }
        float g[K], sum = 0.f;
#pragma unroll
        for (int j = 0; j < K; ++j) { g[j] = __expf(val[j] - val[0]); sum += g[j]; }
        if (live) {
#pragma unroll
            for (int j = 0; j < K; ++j) {
                topk_idx[token * K + j] = idx[j];
                gates[token * K + j] = (T)(g[j] / sum);
            }
            thr_val[token * 2] = val[K - 1];
            thr_val[token * 2 + 1] = val[K];
            thr_idx[token * 2] = idx[K - 1];
            thr_idx[token * 2 + 1] = idx[K];
        }
#pragma unroll
        for (int j = 0; j < K; ++j)
            wave_bins_add(mine, live ? idx[j] : 0, live, match_mask(live ? idx[j] : 0, live, nbits));
        // the smooth load: every lane's P_e, added over the wave
        for (int e = 0; e < n_expert; ++e) {
            float p = 0.f;
            if (live) {
                const float c = (float)clean[row + e];
                const float std_e = softplus_f((float)raw[row + e]) + eps;
                // (an expert is inside when it is one of the K selected: the same rule as the selection's
                // under ties, and independent of how the compiler contracts the two evaluations of noisy)
                bool inside = false;
#pragma unroll
                for (int j = 0; j < K; ++j) inside |= idx[j] == e;
                p = normal_cdf_f((c - (inside ? val[K] : val[K - 1])) / std_e);
            }
#pragma unroll
            for (int off = kWave / 2; off > 0; off >>= 1) p += __shfl_xor(p, off, kWave);
            if (lane_id() == 0) my_load[e] += p;
        }
        wave_lds_sync();
    }
    __syncthreads();
    int32_t *dst = block_hist + (int64_t)blockIdx.x * n_expert;
    float *ldst = load_partial + (int64_t)blockIdx.x * n_expert;
    for (int e = threadIdx.x; e < n_expert; e += kBlock) {
        int32_t c = 0;
        float l = 0.f;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) { c += bins[w * n_expert + e]; l += loads[w * n_expert + e]; }
        dst[e] = c;
        ldst[e] = l;
    }
}

// Backward of the above with respect to the two logit matrices.  Per token, with
// gg_j the gradient of gates_j (the caller has added the importance term) and gl_e that of load_e:
//   d noisy_{i_j} = gates_j (gg_j - sum_i gg_i gates_i)                                      (j < K)
//   dP_e = gl_e phi(z_e):   d clean_e += dP_e / std_e,   d std_e -= dP_e z_e / std_e,
//                           d noisy_{i_K} -= dP_e / std_e (e inside the top K), d noisy_{i_{K-1}} -= ... (outside)
//   d clean_e += d noisy_e,  d std_e += d noisy_e noise_e,  d raw_e = d std_e sigmoid(raw_e)
template <typename T, int K>
__global__ __launch_bounds__(kBlock) void noisy_gate_backward_kernel(
    const T *__restrict__ clean, const T *__restrict__ raw, const T *__restrict__ noise, float eps, int64_t n_tokens,
    int n_expert, const int64_t *__restrict__ topk_idx, const T *__restrict__ gates, const float *__restrict__ thr_val,
    const int32_t *__restrict__ thr_idx, const T *__restrict__ grad_gates, const float *__restrict__ grad_load,
    T *__restrict__ grad_clean, T *__restrict__ grad_raw) {
    const int64_t token = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (token >= n_tokens) return;
    const int64_t row = token * n_expert;
    const float v_out = thr_val[token * 2], v_in = thr_val[token * 2 + 1];
    const int i_out = thr_idx[token * 2], i_in = thr_idx[token * 2 + 1];
    // the gates again in float32 from the selected experts' noisy logits (the stored ones are rounded
    // to the element type, and gg_j - sum_i gg_i gates_i cancels when one gate is close to 1)
    int sel[K];
    float gt[K], dn[K], dot = 0.f, vmax = -__builtin_inff(), gsum = 0.f;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        sel[j] = (int)topk_idx[token * K + j];
        const int e = sel[j] >= 0 && sel[j] < n_expert ? sel[j] : 0;
        gt[j] = (float)clean[row + e] + (float)noise[row + e] * (softplus_f((float)raw[row + e]) + eps);
        vmax = fmaxf(vmax, gt[j]);
    }
#pragma unroll
    for (int j = 0; j < K; ++j) { gt[j] = __expf(gt[j] - vmax); gsum += gt[j]; }
#pragma unroll
    for (int j = 0; j < K; ++j) { gt[j] /= gsum; dot += (float)grad_gates[token * K + j] * gt[j]; }
#pragma unroll
    for (int j = 0; j < K; ++j) dn[j] = gt[j] * ((float)grad_gates[token * K + j] - dot);
    // first pass: what the thresholds collect from every expert's load term
    float s_in = 0.f, s_out = 0.f;
    for (int e = 0; e < n_expert; ++e) {
        const float c = (float)clean[row + e];
        const float std_e = softplus_f((float)raw[row + e]) + eps;
        bool inside = false;
#pragma unroll
        for (int j = 0; j < K; ++j) inside |= sel[j] == e;
        const float z = (c - (inside ? v_in : v_out)) / std_e;
        const float dp = grad_load[e] * 0.39894228040143267794f * __expf(-0.5f * z * z) / std_e;
        if (inside) s_in -= dp; else s_out -= dp;
    }
    for (int e = 0; e < n_expert; ++e) {
        const float c = (float)clean[row + e], r = (float)raw[row + e], nz = (float)noise[row + e];
        const float std_e = softplus_f(r) + eps;
        bool inside = false;
#pragma unroll
        for (int j = 0; j < K; ++j) inside |= sel[j] == e;
        const float z = (c - (inside ? v_in : v_out)) / std_e;
        const float dp = grad_load[e] * 0.39894228040143267794f * __expf(-0.5f * z * z) / std_e;
        float d_noisy = 0.f;
#pragma unroll
        for (int j = 0; j < K; ++j) d_noisy += sel[j] == e ? dn[j] : 0.f;
        if (e == i_in) d_noisy += s_in;
        if (e == i_out) d_noisy += s_out;
        const float d_std = -dp * z + d_noisy * nz;
        grad_clean[row + e] = (T)(dp + d_noisy);
        grad_raw[row + e] = (T)(d_std / (1.f + __expf(-r)));
    }
}

// Gradient of the scores with respect to the logits: zero except at the selected experts.
// score_mode 0: grad_logits[t, idx[t,j]] = grad_score[t,j];
// score_mode 1: grad_logits[t, idx[t,j]] = score[t,j] * (grad_score[t,j] - sum_i grad_score[t,i] score[t,i]).
template <typename T>
__global__ __launch_bounds__(kBlock) void gate_topk_backward_kernel(
    const T *__restrict__ grad_score, const T *__restrict__ score, const int64_t *__restrict__ topk_idx,
    T *__restrict__ grad_logits, int64_t n_tokens, int n_expert, int top_k, int score_mode) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_tokens * n_expert) return;
    const int64_t t = i / n_expert;
    const int e = (int)(i - t * n_expert);
    float dot = 0.f;
    if (score_mode == 1)
        for (int j = 0; j < top_k; ++j) dot += (float)grad_score[t * top_k + j] * (float)score[t * top_k + j];
    float gval = 0.f;
    for (int j = 0; j < top_k; ++j)
        if (topk_idx[t * top_k + j] == e) {
            const float gs = (float)grad_score[t * top_k + j];
            gval = score_mode == 1 ? (float)score[t * top_k + j] * (gs - dot) : gs;
        }
    grad_logits[i] = (T)gval;
}

// ------------------------------------------------------------- capacity ----

// One thread per expert, workers in ascending order (the order that fixes who
// gets the remaining capacity).
__global__ __launch_bounds__(kBlock) void limit_by_capacity_kernel(
    const int64_t *__restrict__ ec, int32_t *__restrict__ cap, int64_t *__restrict__ eca,
    int64_t n_expert, int64_t n_worker) {
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_expert) return;
    int32_t left = cap[e];
    for (int64_t w = 0; w < n_worker; ++w) {
        const int32_t proposal = (int32_t)ec[w * n_expert + e];
        int64_t grant;
        if (left >= proposal) grant = proposal;
        else if (left >= 0) grant = left;
        else grant = 0;
        eca[w * n_expert + e] = grant;
        left -= proposal;
    }
    cap[e] = left;
}

__global__ __launch_bounds__(kBlock) void zero_counts_kernel(int64_t *__restrict__ count, int64_t n) {
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e < n) count[e] = 0;
}

int ilog2_ceil(int64_t n) {
    int b = 0;
    while ((1ll << b) < n) ++b;
    return b < 1 ? 1 : b;
}

// Dynamic LDS beyond 64 KiB (more than 4096 experts) has to be allowed per kernel and device.  The
// opt-in is made once per (kernel, device) and size reached, outside the launch path of later calls
// (so that it does not land inside a stream capture); a failure is reported again by every call.
int allow_lds(const void *kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return FMOE_OK;
    struct Granted { const void *kernel; int device; size_t bytes; bool failed; };
    static std::mutex mutex;
    static Granted granted[64];
    static int n_granted = 0;
    int dev = 0;
    FMOE_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(mutex);
    Granted *slot = nullptr;
    for (int i = 0; i < n_granted; ++i)
        if (granted[i].kernel == kernel && granted[i].device == dev) slot = &granted[i];
    if (slot != nullptr && !slot->failed && slot->bytes >= bytes) return FMOE_OK;
    if (slot == nullptr) {
        FMOE_REQUIRE(n_granted < 64, "too many (kernel, device) pairs ask for more than 64 KiB of LDS");
        slot = &granted[n_granted++];
        *slot = Granted{kernel, dev, 0, false};
    }
    const hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    slot->failed = err != hipSuccess;
    if (!slot->failed) slot->bytes = bytes;
    FMOE_HIP_CHECK(err);
    return FMOE_OK;
}

struct RouteScratch {
    int32_t *block_hist;  // [n_blocks][n_expert]
    int32_t *limit_old;   // [n_expert]
    int32_t *cum;         // [n_expert]  (fmoe_route only)
    int n_blocks;
};

int64_t scratch_bytes(int64_t n_slots, int64_t n_expert) {
    const int64_t nb = ceil_div(n_slots > 0 ? n_slots : 1, kSlotsPerBlock);
    return (nb * n_expert + 2 * n_expert) * (int64_t)sizeof(int32_t) + 64;
}

int carve(void *workspace, int64_t workspace_bytes, int64_t n_slots, int64_t n_expert, RouteScratch *s) {
    const int64_t need = scratch_bytes(n_slots, n_expert);
    if (workspace == nullptr || workspace_bytes < need)
        return fail(FMOE_EWORKSPACE, "routing workspace: need %lld bytes, got %lld",
                    (long long)need, (long long)workspace_bytes);
    FMOE_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 3u) == 0, "routing workspace must be 4-byte aligned");
    const int64_t nb = ceil_div(n_slots > 0 ? n_slots : 1, kSlotsPerBlock);
    s->block_hist = static_cast<int32_t *>(workspace);
    s->limit_old = s->block_hist + nb * n_expert;
    s->cum = s->limit_old + n_expert;
    s->n_blocks = (int)nb;
    return FMOE_OK;
}

int check_sizes(int64_t n_slots, int64_t n_expert) {
    FMOE_REQUIRE(n_slots >= 0, "n_slots must be >= 0 (got %lld)", (long long)n_slots);
    FMOE_REQUIRE(n_expert >= 1, "n_expert must be >= 1 (got %lld)", (long long)n_expert);
    if (n_expert > kMaxExpert)
        return fail(FMOE_ELIMIT, "n_expert %lld exceeds the supported maximum %lld",
                    (long long)n_expert, (long long)kMaxExpert);
    if (n_slots > (int64_t)INT32_MAX)
        return fail(FMOE_ELIMIT, "n_slots %lld exceeds int32 range", (long long)n_slots);
    return FMOE_OK;
}

}  // namespace
}  // namespace fmoe

using namespace fmoe;

extern "C" int fmoe_expert_count(const int64_t *gate_idx, int32_t *expert_count, int64_t n_slots,
                                 int64_t n_expert, void *stream) {
    if (int rc = check_sizes(n_slots, n_expert)) return rc;
    if (n_slots == 0) return FMOE_OK;
    FMOE_REQUIRE(gate_idx && expert_count, "fmoe_expert_count: NULL pointer");
    const int64_t blocks = ceil_div(n_slots, (int64_t)kBlock * 8);
    const int grid = (int)(blocks < 1024 ? blocks : 1024);
    const size_t lds = kWavesPerBlock * n_expert * sizeof(int32_t);
    if (int rc = allow_lds((const void *)expert_count_kernel, lds)) return rc;
    expert_count_kernel<<<grid, kBlock, lds, (hipStream_t)stream>>>(
        gate_idx, expert_count, n_slots, (int)n_expert, ilog2_ceil(n_expert));
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

extern "C" int64_t fmoe_routing_workspace_bytes(int64_t n_slots, int64_t n_expert) {
    if (n_slots < 0 || n_expert < 1) return 0;
    return scratch_bytes(n_slots, n_expert);
}

extern "C" int fmoe_assign_pos(int32_t *cum_count, const int64_t *gate, int64_t *pos, int64_t n_pos,
                               int64_t n_slots, int64_t n_expert, void *workspace, int64_t workspace_bytes,
                               void *stream) {
    if (int rc = check_sizes(n_slots, n_expert)) return rc;
    if (n_slots == 0) return FMOE_OK;
    FMOE_REQUIRE(cum_count && gate && n_pos >= 0 && (pos || n_pos == 0), "fmoe_assign_pos: NULL pointer");
    RouteScratch s;
    if (int rc = carve(workspace, workspace_bytes, n_slots, n_expert, &s)) return rc;
    hipStream_t st = (hipStream_t)stream;
    const int E = (int)n_expert;
    if (int rc = allow_lds((const void *)block_hist_kernel, kWavesPerBlock * E * sizeof(int32_t))) return rc;
    block_hist_kernel<<<s.n_blocks, kBlock, kWavesPerBlock * E * sizeof(int32_t), st>>>(gate, s.block_hist, n_slots, E, ilog2_ceil(n_expert));
    FMOE_LAUNCH_CHECK();
    block_scan_kernel<<<(int)ceil_div(E, kBlock), kBlock, 0, st>>>(s.block_hist, s.n_blocks, E, cum_count, s.limit_old);
    FMOE_LAUNCH_CHECK();
    if (int rc = allow_lds((const void *)rank_apply_kernel<kApplyAssign>, kWavesPerBlock * E * sizeof(int32_t))) return rc;
    rank_apply_kernel<kApplyAssign><<<s.n_blocks, kBlock, kWavesPerBlock * E * sizeof(int32_t), st>>>(
        gate, s.block_hist, s.limit_old, pos, nullptr, n_slots, n_pos, E, ilog2_ceil(n_expert), 0);
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

namespace fmoe {
namespace {

// histogram -> scan over workgroups and experts -> placement, on scratch carved by the caller
int route_launch(const int64_t *gate, int64_t n_slots, int64_t n_expert, int64_t *expert_count, int64_t *pos,
                 int64_t *slot_to_row, const RouteScratch &s, hipStream_t st) {
    const int E = (int)n_expert;
    if (int rc = allow_lds((const void *)block_hist_kernel, kWavesPerBlock * E * sizeof(int32_t))) return rc;
    block_hist_kernel<<<s.n_blocks, kBlock, kWavesPerBlock * E * sizeof(int32_t), st>>>(gate, s.block_hist, n_slots, E, ilog2_ceil(n_expert));
    FMOE_LAUNCH_CHECK();
    route_scan_kernel<<<1, kRouteScanBlock, 0, st>>>(s.block_hist, s.n_blocks, E, expert_count, s.cum);
    FMOE_LAUNCH_CHECK();
    if (int rc = allow_lds((const void *)rank_apply_kernel<kApplyAssign>, kWavesPerBlock * E * sizeof(int32_t))) return rc;
    rank_apply_kernel<kApplyAssign><<<s.n_blocks, kBlock, kWavesPerBlock * E * sizeof(int32_t), st>>>(
        gate, s.block_hist, s.cum, pos, slot_to_row, n_slots, n_slots, E, ilog2_ceil(n_expert), 1);
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

int route_empty(int64_t n_expert, int64_t *expert_count, hipStream_t st) {
    // a fill kernel, not hipMemsetAsync, so that the call can be captured into a HIP graph
    zero_counts_kernel<<<(int)ceil_div(n_expert, kBlock), kBlock, 0, st>>>(expert_count, n_expert);
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

// Scratch of fmoe_route_static: a fixed device array instead of a caller's workspace, so
// that the entry point never allocates.  Every GPU holds its own copy at its own address;
// `scratch` is only the host-side handle of the symbol, the device address is looked
// up once per device and kept in g_static_scratch_ptr.
constexpr int64_t kStaticScratchBytes = FMOE_ROUTE_STATIC_SCRATCH_BYTES;
constexpr int kMaxDevices = 16;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
std::mutex g_static_scratch_mutex;
void *g_static_scratch_ptr[kMaxDevices] = {};

int static_scratch_address(void **out) {
    int dev = 0;
    FMOE_HIP_CHECK(hipGetDevice(&dev));
    FMOE_REQUIRE(dev >= 0 && dev < kMaxDevices, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (g_static_scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        FMOE_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        FMOE_REQUIRE(ptr != nullptr, "hipGetSymbolAddress returned NULL for the routing scratch");
        g_static_scratch_ptr[dev] = ptr;
    }
    *out = g_static_scratch_ptr[dev];
    return FMOE_OK;
}

}  // namespace
}  // namespace fmoe

extern "C" int fmoe_route(const int64_t *gate, int64_t n_slots, int64_t n_expert, int64_t *expert_count,
                          int64_t *pos, int64_t *slot_to_row, void *workspace, int64_t workspace_bytes,
                          void *stream) {
    if (int rc = check_sizes(n_slots, n_expert)) return rc;
    FMOE_REQUIRE(expert_count, "fmoe_route: NULL expert_count");
    hipStream_t st = (hipStream_t)stream;
    if (n_slots == 0) return route_empty(n_expert, expert_count, st);
    FMOE_REQUIRE(gate && pos, "fmoe_route: NULL pointer");
    RouteScratch s;
    if (int rc = carve(workspace, workspace_bytes, n_slots, n_expert, &s)) return rc;
    return route_launch(gate, n_slots, n_expert, expert_count, pos, slot_to_row, s, st);
}

extern "C" int fmoe_route_static(const int64_t *gate, int64_t n_slots, int64_t n_expert, int64_t *expert_count,
                                 int64_t *pos, int64_t *slot_to_row, void *stream) {
    if (int rc = check_sizes(n_slots, n_expert)) return rc;
    FMOE_REQUIRE(expert_count, "fmoe_route_static: NULL expert_count");
    hipStream_t st = (hipStream_t)stream;
    if (n_slots == 0) return route_empty(n_expert, expert_count, st);
    FMOE_REQUIRE(gate && pos, "fmoe_route_static: NULL pointer");
    const int64_t need = scratch_bytes(n_slots, n_expert);
    if (need > kStaticScratchBytes)
        return fail(FMOE_ELIMIT,
                    "fmoe_route_static: %lld slots x %lld experts need %lld bytes of scratch, the built-in "
                    "array holds %lld; use fmoe_route with a workspace",
                    (long long)n_slots, (long long)n_expert, (long long)need, (long long)kStaticScratchBytes);
    void *scratch_dev = nullptr;
    if (int rc = static_scratch_address(&scratch_dev)) return rc;
    RouteScratch s;
    if (int rc = carve(scratch_dev, kStaticScratchBytes, n_slots, n_expert, &s)) return rc;
    // Every cell of the scratch that the scan and the placement read is written by the
    // histogram / scan launched just before them, so nothing has to be cleared between calls.
    return route_launch(gate, n_slots, n_expert, expert_count, pos, slot_to_row, s, st);
}

extern "C" int fmoe_limit_by_capacity(const int64_t *ec, int32_t *cap, int64_t *eca, int64_t n_expert,
                                      int64_t n_worker, void *stream) {
    FMOE_REQUIRE(n_expert >= 1 && n_worker >= 1, "fmoe_limit_by_capacity: n_expert=%lld n_worker=%lld",
                 (long long)n_expert, (long long)n_worker);
    FMOE_REQUIRE(ec && cap && eca, "fmoe_limit_by_capacity: NULL pointer");
    limit_by_capacity_kernel<<<(int)ceil_div(n_expert, kBlock), kBlock, 0, (hipStream_t)stream>>>(
        ec, cap, eca, n_expert, n_worker);
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

extern "C" int fmoe_prune_gate_by_capacity(const int64_t *gate_idx, int64_t *new_gate_idx, int32_t *ec,
                                           int64_t n_slots, int64_t n_expert, void *workspace,
                                           int64_t workspace_bytes, void *stream) {
    if (int rc = check_sizes(n_slots, n_expert)) return rc;
    if (n_slots == 0) return FMOE_OK;
    FMOE_REQUIRE(gate_idx && new_gate_idx && ec, "fmoe_prune_gate_by_capacity: NULL pointer");
    RouteScratch s;
    if (int rc = carve(workspace, workspace_bytes, n_slots, n_expert, &s)) return rc;
    hipStream_t st = (hipStream_t)stream;
    const int E = (int)n_expert;
    if (int rc = allow_lds((const void *)block_hist_kernel, kWavesPerBlock * E * sizeof(int32_t))) return rc;
    block_hist_kernel<<<s.n_blocks, kBlock, kWavesPerBlock * E * sizeof(int32_t), st>>>(gate_idx, s.block_hist, n_slots, E, ilog2_ceil(n_expert));
    FMOE_LAUNCH_CHECK();
    block_scan_kernel<<<(int)ceil_div(E, kBlock), kBlock, 0, st>>>(s.block_hist, s.n_blocks, E, ec, s.limit_old);
    FMOE_LAUNCH_CHECK();
    if (int rc = allow_lds((const void *)rank_apply_kernel<kApplyPrune>, kWavesPerBlock * E * sizeof(int32_t))) return rc;
    rank_apply_kernel<kApplyPrune><<<s.n_blocks, kBlock, kWavesPerBlock * E * sizeof(int32_t), st>>>(
        gate_idx, s.block_hist, s.limit_old, new_gate_idx, nullptr, n_slots, n_slots, E, ilog2_ceil(n_expert), 0);
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}


namespace fmoe {
namespace {

template <typename T>
int launch_gate_topk(const void *logits, int64_t n_tokens, int E, int top_k, int score_mode, int64_t *topk_idx,
                     void *topk_score, int32_t *block_hist, int n_blocks, hipStream_t st) {
    const size_t lds = kWavesPerBlock * E * sizeof(int32_t);
    const int nbits = ilog2_ceil(E);
    // rows start on 16-byte boundaries: vector loads
    const int vector_rows = (E * sizeof(T)) % 16 == 0 && (reinterpret_cast<uintptr_t>(logits) & 15u) == 0;
#define FMOE_GATE_LAUNCH(KK)                                                                                      \
    do {                                                                                                          \
        if (int rc = allow_lds((const void *)gate_topk_hist_kernel<T, KK>, lds)) return rc;                       \
        gate_topk_hist_kernel<T, KK><<<n_blocks, kBlock, lds, st>>>((const T *)logits, n_tokens, E, score_mode,   \
                                                                    vector_rows, topk_idx, (T *)topk_score,       \
                                                                    block_hist, nbits);                           \
    } while (0)
    switch (top_k) {
        case 1: FMOE_GATE_LAUNCH(1); break;
        case 2: FMOE_GATE_LAUNCH(2); break;
        case 4: FMOE_GATE_LAUNCH(4); break;
        case 8: FMOE_GATE_LAUNCH(8); break;
        default: return fail(FMOE_ELIMIT, "gate top-k: top_k=%d is not 1, 2, 4 or 8", top_k);
    }
#undef FMOE_GATE_LAUNCH
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

}  // namespace
}  // namespace fmoe

extern "C" int fmoe_gate_topk_route(const void *logits, int64_t n_tokens, int64_t n_expert, int64_t top_k, int dtype,
                                    int score_mode, int64_t *topk_idx, void *topk_score, int64_t *expert_count,
                                    int64_t *pos, int64_t *slot_to_row, void *workspace, int64_t workspace_bytes,
                                    void *stream) {
    FMOE_REQUIRE(n_tokens >= 0 && top_k >= 1, "fmoe_gate_topk_route: n_tokens=%lld top_k=%lld", (long long)n_tokens,
                 (long long)top_k);
    FMOE_REQUIRE(dtype == FMOE_F32 || dtype == FMOE_BF16 || dtype == FMOE_F16, "fmoe_gate_topk_route: dtype %d", dtype);
    FMOE_REQUIRE(score_mode == 0 || score_mode == 1, "fmoe_gate_topk_route: score_mode %d", score_mode);
    if (top_k > n_expert || (top_k != 1 && top_k != 2 && top_k != 4 && top_k != 8))
        return fail(FMOE_ELIMIT, "fmoe_gate_topk_route: top_k=%lld must be 1, 2, 4 or 8 and at most n_expert",
                    (long long)top_k);
    const int64_t n_slots = n_tokens * top_k;
    if (int rc = check_sizes(n_slots, n_expert)) return rc;
    FMOE_REQUIRE(expert_count, "fmoe_gate_topk_route: NULL expert_count");
    hipStream_t st = (hipStream_t)stream;
    if (n_slots == 0) return route_empty(n_expert, expert_count, st);
    FMOE_REQUIRE(logits && topk_idx && topk_score && pos, "fmoe_gate_topk_route: NULL pointer");
    RouteScratch s;
    if (int rc = carve(workspace, workspace_bytes, n_slots, n_expert, &s)) return rc;
    const int E = (int)n_expert;
    int rc = FMOE_OK;
    switch (dtype) {
        case FMOE_F32: rc = launch_gate_topk<float>(logits, n_tokens, E, (int)top_k, score_mode, topk_idx, topk_score, s.block_hist, s.n_blocks, st); break;
        case FMOE_BF16: rc = launch_gate_topk<__bf16>(logits, n_tokens, E, (int)top_k, score_mode, topk_idx, topk_score, s.block_hist, s.n_blocks, st); break;
        default: rc = launch_gate_topk<_Float16>(logits, n_tokens, E, (int)top_k, score_mode, topk_idx, topk_score, s.block_hist, s.n_blocks, st); break;
    }
    if (rc) return rc;
    route_scan_kernel<<<1, kRouteScanBlock, 0, st>>>(s.block_hist, s.n_blocks, E, expert_count, s.cum);
    FMOE_LAUNCH_CHECK();
    if (int rc2 = allow_lds((const void *)rank_apply_kernel<kApplyAssign>, kWavesPerBlock * E * sizeof(int32_t))) return rc2;
    rank_apply_kernel<kApplyAssign><<<s.n_blocks, kBlock, kWavesPerBlock * E * sizeof(int32_t), st>>>(
        topk_idx, s.block_hist, s.cum, pos, slot_to_row, n_slots, n_slots, E, ilog2_ceil(n_expert), 1);
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

namespace fmoe {
namespace {

template <typename T>
int launch_gate_linear(const void *x, const void *w, const void *bias, int64_t n_tokens, int d, int E, int top_k,
                       int score_mode, int64_t *topk_idx, void *topk_score, hipStream_t st) {
    const unsigned grid = (unsigned)ceil_div(n_tokens, kGateTokens);
    const size_t lds = (size_t)kWavesPerBlock * ((E + 15) / 16 * 16) * kGateStride * sizeof(float);
    // (accumulators for 1, 2 or 4 blocks of 16 experts: fewer registers, more waves per compute unit)
#define FMOE_GATE_LINEAR_LAUNCH(KK)                                                                                         \
    do {                                                                                                                    \
        if (E <= 16)                                                                                                        \
            gate_linear_topk_kernel<T, KK, 1><<<grid, kBlock, lds, st>>>((const T *)x, (const T *)w, (const T *)bias,        \
                                                                         n_tokens, d, E, score_mode, topk_idx, (T *)topk_score); \
        else if (E <= 32)                                                                                                   \
            gate_linear_topk_kernel<T, KK, 2><<<grid, kBlock, lds, st>>>((const T *)x, (const T *)w, (const T *)bias,        \
                                                                         n_tokens, d, E, score_mode, topk_idx, (T *)topk_score); \
        else                                                                                                                \
            gate_linear_topk_kernel<T, KK, 4><<<grid, kBlock, lds, st>>>((const T *)x, (const T *)w, (const T *)bias,        \
                                                                         n_tokens, d, E, score_mode, topk_idx, (T *)topk_score); \
    } while (0)
    switch (top_k) {
        case 1: FMOE_GATE_LINEAR_LAUNCH(1); break;
        case 2: FMOE_GATE_LINEAR_LAUNCH(2); break;
        case 4: FMOE_GATE_LINEAR_LAUNCH(4); break;
        case 8: FMOE_GATE_LINEAR_LAUNCH(8); break;
        default: return fail(FMOE_ELIMIT, "gate linear top-k: top_k=%d is not 1, 2, 4 or 8", top_k);
    }
#undef FMOE_GATE_LINEAR_LAUNCH
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

}  // namespace
}  // namespace fmoe

extern "C" int fmoe_gate_linear_supported(int64_t d_model, int64_t n_expert, int64_t top_k, int dtype) {
    if (dtype != FMOE_F32 && dtype != FMOE_BF16 && dtype != FMOE_F16) return 0;
    if (n_expert < 1 || n_expert > kGateMaxExpert || top_k > n_expert) return 0;
    if (top_k != 1 && top_k != 2 && top_k != 4 && top_k != 8) return 0;
    return (d_model >= 1 && d_model < (1 << 30) && (d_model * dtype_bytes(dtype)) % 16 == 0) ? 1 : 0;
}

extern "C" int fmoe_gate_linear_topk_route(const void *x, const void *w, const void *bias, int64_t n_tokens,
                                           int64_t d_model, int64_t n_expert, int64_t top_k, int dtype, int score_mode,
                                           int64_t *topk_idx, void *topk_score, int64_t *expert_count, int64_t *pos,
                                           int64_t *slot_to_row, void *workspace, int64_t workspace_bytes,
                                           void *stream) {
    FMOE_REQUIRE(n_tokens >= 0 && top_k >= 1, "fmoe_gate_linear_topk_route: n_tokens=%lld top_k=%lld",
                 (long long)n_tokens, (long long)top_k);
    FMOE_REQUIRE(score_mode == 0 || score_mode == 1, "fmoe_gate_linear_topk_route: score_mode %d", score_mode);
    if (!fmoe_gate_linear_supported(d_model, n_expert, top_k, dtype))
        return fail(FMOE_ELIMIT,
                    "fmoe_gate_linear_topk_route: d_model=%lld n_expert=%lld top_k=%lld dtype=%d is not taken (at most %d "
                    "experts, top_k 1, 2, 4 or 8, rows of whole 16-byte chunks, 16- or 32-bit floats)",
                    (long long)d_model, (long long)n_expert, (long long)top_k, dtype, kGateMaxExpert);
    const int64_t n_slots = n_tokens * top_k;
    if (int rc = check_sizes(n_slots, n_expert)) return rc;
    FMOE_REQUIRE(expert_count, "fmoe_gate_linear_topk_route: NULL expert_count");
    hipStream_t st = (hipStream_t)stream;
    if (n_slots == 0) return route_empty(n_expert, expert_count, st);
    FMOE_REQUIRE(x && w && topk_idx && topk_score && pos, "fmoe_gate_linear_topk_route: NULL pointer");
    FMOE_REQUIRE(aligned16(x) && aligned16(w), "fmoe_gate_linear_topk_route: x and w must be 16-byte aligned");
    RouteScratch s;
    if (int rc = carve(workspace, workspace_bytes, n_slots, n_expert, &s)) return rc;
    int rc = FMOE_OK;
    switch (dtype) {
        case FMOE_F32: rc = launch_gate_linear<float>(x, w, bias, n_tokens, (int)d_model, (int)n_expert, (int)top_k, score_mode, topk_idx, topk_score, st); break;
        case FMOE_BF16: rc = launch_gate_linear<__bf16>(x, w, bias, n_tokens, (int)d_model, (int)n_expert, (int)top_k, score_mode, topk_idx, topk_score, st); break;
        default: rc = launch_gate_linear<_Float16>(x, w, bias, n_tokens, (int)d_model, (int)n_expert, (int)top_k, score_mode, topk_idx, topk_score, st); break;
    }
    if (rc) return rc;
    return route_launch(topk_idx, n_slots, n_expert, expert_count, pos, slot_to_row, s, st);
}

extern "C" int fmoe_noisy_gate_forward(const void *clean, const void *raw, const void *noise, double eps,
                                       int64_t n_tokens, int64_t n_expert, int64_t top_k, int dtype,
                                       int64_t *topk_idx, void *gates, float *thr_val, int32_t *thr_idx,
                                       float *load_partial, int64_t *expert_count, int64_t *pos, int64_t *slot_to_row,
                                       void *workspace, int64_t workspace_bytes, void *stream) {
    FMOE_REQUIRE(n_tokens >= 0 && top_k >= 1, "fmoe_noisy_gate_forward: n_tokens=%lld top_k=%lld", (long long)n_tokens,
                 (long long)top_k);
    FMOE_REQUIRE(dtype == FMOE_F32 || dtype == FMOE_BF16 || dtype == FMOE_F16, "fmoe_noisy_gate_forward: dtype %d", dtype);
    if (top_k >= n_expert || (top_k != 1 && top_k != 2 && top_k != 4 && top_k != 8) || n_expert > 2048)
        return fail(FMOE_ELIMIT, "fmoe_noisy_gate_forward: top_k=%lld must be 1, 2, 4 or 8 and below n_expert=%lld <= 2048",
                    (long long)top_k, (long long)n_expert);
    const int64_t n_slots = n_tokens * top_k;
    if (int rc = check_sizes(n_slots, n_expert)) return rc;
    FMOE_REQUIRE(expert_count && load_partial, "fmoe_noisy_gate_forward: NULL expert_count / load_partial");
    hipStream_t st = (hipStream_t)stream;
    if (n_slots == 0) return route_empty(n_expert, expert_count, st);
    FMOE_REQUIRE(clean && raw && noise && topk_idx && gates && thr_val && thr_idx && pos,
                 "fmoe_noisy_gate_forward: NULL pointer");
    RouteScratch s;
    if (int rc = carve(workspace, workspace_bytes, n_slots, n_expert, &s)) return rc;
    const int E = (int)n_expert, nbits = ilog2_ceil(n_expert);
    const size_t lds = 2 * kWavesPerBlock * E * sizeof(int32_t);
#define FMOE_NOISY_FWD(TT, KK)                                                                                          \
    do {                                                                                                                \
        if (int rc = allow_lds((const void *)noisy_gate_forward_kernel<TT, KK>, lds)) return rc;                        \
        noisy_gate_forward_kernel<TT, KK><<<s.n_blocks, kBlock, lds, st>>>(                                             \
            (const TT *)clean, (const TT *)raw, (const TT *)noise, (float)eps, n_tokens, E, topk_idx, (TT *)gates,      \
            thr_val, thr_idx, load_partial, s.block_hist, nbits);                                                       \
    } while (0)
#define FMOE_NOISY_FWD_K(TT)                                                 \
    switch (top_k) {                                                         \
        case 1: FMOE_NOISY_FWD(TT, 1); break;                                \
        case 2: FMOE_NOISY_FWD(TT, 2); break;                                \
        case 4: FMOE_NOISY_FWD(TT, 4); break;                                \
        default: FMOE_NOISY_FWD(TT, 8); break;                               \
    }
    switch (dtype) {
        case FMOE_F32: FMOE_NOISY_FWD_K(float); break;
        case FMOE_BF16: FMOE_NOISY_FWD_K(__bf16); break;
        default: FMOE_NOISY_FWD_K(_Float16); break;
    }
#undef FMOE_NOISY_FWD_K
#undef FMOE_NOISY_FWD
    FMOE_LAUNCH_CHECK();
    route_scan_kernel<<<1, kRouteScanBlock, 0, st>>>(s.block_hist, s.n_blocks, E, expert_count, s.cum);
    FMOE_LAUNCH_CHECK();
    if (int rc2 = allow_lds((const void *)rank_apply_kernel<kApplyAssign>, kWavesPerBlock * E * sizeof(int32_t))) return rc2;
    rank_apply_kernel<kApplyAssign><<<s.n_blocks, kBlock, kWavesPerBlock * E * sizeof(int32_t), st>>>(
        topk_idx, s.block_hist, s.cum, pos, slot_to_row, n_slots, n_slots, E, nbits, 1);
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

extern "C" int fmoe_noisy_gate_backward(const void *clean, const void *raw, const void *noise, double eps,
                                        int64_t n_tokens, int64_t n_expert, int64_t top_k, int dtype,
                                        const int64_t *topk_idx, const void *gates, const float *thr_val,
                                        const int32_t *thr_idx, const void *grad_gates, const float *grad_load,
                                        void *grad_clean, void *grad_raw, void *stream) {
    FMOE_REQUIRE(n_tokens >= 0 && n_expert >= 1, "fmoe_noisy_gate_backward: bad sizes");
    FMOE_REQUIRE(dtype == FMOE_F32 || dtype == FMOE_BF16 || dtype == FMOE_F16, "fmoe_noisy_gate_backward: dtype %d", dtype);
    if (top_k >= n_expert || (top_k != 1 && top_k != 2 && top_k != 4 && top_k != 8))
        return fail(FMOE_ELIMIT, "fmoe_noisy_gate_backward: top_k=%lld", (long long)top_k);
    if (n_tokens == 0) return FMOE_OK;
    FMOE_REQUIRE(clean && raw && noise && topk_idx && gates && thr_val && thr_idx && grad_gates && grad_load &&
                     grad_clean && grad_raw, "fmoe_noisy_gate_backward: NULL pointer");
    hipStream_t st = (hipStream_t)stream;
    const unsigned grid = (unsigned)ceil_div(n_tokens, kBlock);
    const int E = (int)n_expert;
#define FMOE_NOISY_BWD(TT, KK)                                                                                            \
    noisy_gate_backward_kernel<TT, KK><<<grid, kBlock, 0, st>>>((const TT *)clean, (const TT *)raw, (const TT *)noise,   \
                                                               (float)eps, n_tokens, E, topk_idx, (const TT *)gates,    \
                                                               thr_val, thr_idx, (const TT *)grad_gates, grad_load,     \
                                                               (TT *)grad_clean, (TT *)grad_raw)
#define FMOE_NOISY_BWD_K(TT)                                                 \
    switch (top_k) {                                                         \
        case 1: FMOE_NOISY_BWD(TT, 1); break;                                \
        case 2: FMOE_NOISY_BWD(TT, 2); break;                                \
        case 4: FMOE_NOISY_BWD(TT, 4); break;                                \
        default: FMOE_NOISY_BWD(TT, 8); break;                               \
    }
    switch (dtype) {
        case FMOE_F32: FMOE_NOISY_BWD_K(float); break;
        case FMOE_BF16: FMOE_NOISY_BWD_K(__bf16); break;
        default: FMOE_NOISY_BWD_K(_Float16); break;
    }
#undef FMOE_NOISY_BWD_K
#undef FMOE_NOISY_BWD
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}

extern "C" int fmoe_gate_topk_backward(const void *grad_score, const void *score, const int64_t *topk_idx,
                                       void *grad_logits, int64_t n_tokens, int64_t n_expert, int64_t top_k,
                                       int dtype, int score_mode, void *stream) {
    FMOE_REQUIRE(n_tokens >= 0 && n_expert >= 1 && top_k >= 1, "fmoe_gate_topk_backward: bad sizes");
    FMOE_REQUIRE(dtype == FMOE_F32 || dtype == FMOE_BF16 || dtype == FMOE_F16, "fmoe_gate_topk_backward: dtype %d", dtype);
    FMOE_REQUIRE(score_mode == 0 || score_mode == 1, "fmoe_gate_topk_backward: score_mode %d", score_mode);
    const int64_t n = n_tokens * n_expert;
    if (n == 0) return FMOE_OK;
    if (n > (int64_t)INT32_MAX * kBlock) return fail(FMOE_ELIMIT, "fmoe_gate_topk_backward: %lld logits", (long long)n);
    FMOE_REQUIRE(grad_score && topk_idx && grad_logits && (score_mode == 0 || score), "fmoe_gate_topk_backward: NULL pointer");
    const unsigned grid = (unsigned)ceil_div(n, kBlock);
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FMOE_F32: gate_topk_backward_kernel<float><<<grid, kBlock, 0, st>>>((const float *)grad_score, (const float *)score, topk_idx, (float *)grad_logits, n_tokens, (int)n_expert, (int)top_k, score_mode); break;
        case FMOE_BF16: gate_topk_backward_kernel<__bf16><<<grid, kBlock, 0, st>>>((const __bf16 *)grad_score, (const __bf16 *)score, topk_idx, (__bf16 *)grad_logits, n_tokens, (int)n_expert, (int)top_k, score_mode); break;
        default: gate_topk_backward_kernel<_Float16><<<grid, kBlock, 0, st>>>((const _Float16 *)grad_score, (const _Float16 *)score, topk_idx, (_Float16 *)grad_logits, n_tokens, (int)n_expert, (int)top_k, score_mode); break;
    }
    FMOE_LAUNCH_CHECK();
    return FMOE_OK;
}
