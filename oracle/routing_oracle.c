/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's routing and
 * capacity kernels.  Nothing in the product path may link, load or call this
 * file; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do,
 * and only as the checker.
 *
 * The reference kernels use atomicSub/atomicAdd, so their result depends on the
 * order in which threads reach the atomic.  The canonical order fixed here is
 * "one thread at a time, in ascending flat index", i.e. what the kernel gives
 * when executed sequentially.  Every function below is that sequential
 * execution, written as a plain loop.
 *
 * Pinning (see tests/test_oracle.py): expert_count against numpy.bincount;
 * assign_pos against a stable-argsort closed form and the schedule-independent
 * invariants (permutation of valid slots, non-decreasing expert along pos,
 * segment bounds); limit_by_capacity against min(count, cap) at one worker and
 * a hand-worked 3-worker case; prune_gate_by_capacity against the
 * rank-within-expert closed form and the surviving-count <= capacity invariant
 * of the reference's tests/test_gates.py:51-57.
 */
#include <stdint.h>

/* cuda/local_exchange.cuh:32-61 (expert_count_kernel): histogram of gate
 * indices, -1 skipped, result ADDED to expert_count (the caller zero-fills,
 * fmoe/functions.py:21-24).  Indices outside [0, n_expert) are skipped, as the
 * kernel's expert_min/expert_max window does. */
void oracle_expert_count(const int64_t *gate_idx, int32_t *expert_count,
                         int64_t n_slots, int64_t n_expert)
{
    for (int64_t i = 0; i < n_slots; ++i) {
        int64_t g = gate_idx[i];
        if (g < 0 || g >= n_expert)
            continue;
        expert_count[g] += 1;
    }
}

/* cuda/local_exchange.cuh:5-16 (assign_pos_kernel): for each slot with
 * gate > -1, p = atomicSub(&cum_count[gate], 1); pos[p - 1] = idx.
 * cum_count enters as the inclusive cumsum of the counts and leaves as the
 * exclusive one.  Sequential execution puts the slots of one expert in
 * DESCENDING flat index inside the expert's segment. */
void oracle_assign_pos(int32_t *cum_count, const int64_t *gate, int64_t *pos,
                       int64_t n_slots)
{
    for (int64_t idx = 0; idx < n_slots; ++idx) {
        int64_t g = gate[idx];
        if (g > -1) {
            int32_t p = cum_count[g];
            cum_count[g] = p - 1;
            pos[p - 1] = idx;
        }
    }
}

/* cuda/balancing.cuh:5-21 (limit_by_capacity_kernel): worker w asks expert e
 * for ec[w,e] slots; cap[e] is decremented by the proposal whatever the
 * outcome; the grant is the proposal, what was left, or 0.  The proposal is
 * truncated to int as in the kernel (balancing.cuh:11).  Sequential order:
 * workers ascending for each expert. */
void oracle_limit_by_capacity(const int64_t *ec, int32_t *cap, int64_t *eca,
                              int64_t n_expert, int64_t n_worker)
{
    for (int64_t e = 0; e < n_expert; ++e) {
        for (int64_t w = 0; w < n_worker; ++w) {
            int32_t proposal = (int32_t)ec[w * n_expert + e];
            int32_t cap_left = cap[e];
            cap[e] = cap_left - proposal;
            int64_t grant;
            if (cap_left >= proposal)
                grant = proposal;
            else if (cap_left >= 0)
                grant = cap_left;
            else
                grant = 0;
            eca[w * n_expert + e] = grant;
        }
    }
}

/* cuda/balancing.cuh:33-46 (prune_gate_by_capacity_kernel): every slot takes
 * one unit of its expert's remaining capacity; slots that find none left are
 * rewritten to -1.  ec is decremented for every slot, kept or not.  The
 * reference does not guard against a -1 already in the input (it would index
 * ec[-1]); here such a slot stays -1 and takes no capacity. */
void oracle_prune_gate_by_capacity(const int64_t *gate_idx,
                                   int64_t *new_gate_idx, int32_t *ec,
                                   int64_t n_slots)
{
    for (int64_t i = 0; i < n_slots; ++i) {
        int64_t g = gate_idx[i];
        if (g < 0) {
            new_gate_idx[i] = -1;
            continue;
        }
        int32_t orig_cap = ec[g];
        ec[g] = orig_cap - 1;
        new_gate_idx[i] = (orig_cap <= 0) ? -1 : g;
    }
}
