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
        auto insert = [&](float x, int e) {
#pragma unroll
            for (int j = K - 1; j >= 0; --j) {
                const bool here = x > val[j];                       // x belongs at or above place j
                const bool above = j > 0 && x > val[j > 0 ? j - 1 : 0];  // ... above it: place j takes its upper neighbour
                val[j] = here ? (above ? val[j > 0 ? j - 1 : 0] : x) : val[j];
                idx[j] = here ? (above ? idx[j > 0 ? j - 1 : 0] : e) : idx[j];
            }
        };
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

// Dynamic LDS beyond 64 KiB (more than 4096 experts) has to be allowed per kernel.
int allow_lds(const void *kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return FMOE_OK;
    FMOE_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
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
