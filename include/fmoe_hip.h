/*
 * fmoe_hip.h -- C ABI of libfmoe_hip.so, the gfx950 (MI355X) kernels behind the
 * fmoe Python API's single-GPU MoE path.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     all work is enqueued on it and nothing synchronises with the host;
 *   - every entry point returns 0 on success and a negative FMOE_E* code on
 *     failure; fmoe_last_error() then holds a message for the calling thread;
 *   - inputs are borrowed, outputs are caller-allocated, nothing is freed here;
 *   - tensors are dense row-major.
 *
 * Each entry point names the reference interface (thu-pacman/FasterMoE) it
 * stands in for.
 */
#ifndef FMOE_HIP_H
#define FMOE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FMOE_OK 0
#define FMOE_EINVAL (-1)    /* bad argument (shape, alignment, dtype, NULL) */
#define FMOE_ELIMIT (-2)    /* size beyond what the kernels support */
#define FMOE_EHIP (-3)      /* a HIP runtime call failed */
#define FMOE_EWORKSPACE (-4) /* workspace missing or too small */

/* element types of activation / weight tensors */
#define FMOE_F32 0
#define FMOE_BF16 1
#define FMOE_F16 2
#define FMOE_F64 3

/* activation between the two expert linears of the fused MLP */
#define FMOE_ACT_NONE 0
#define FMOE_ACT_RELU 1
#define FMOE_ACT_GELU 2 /* exact erf form, torch.nn.GELU() default */

const char *fmoe_last_error(void);
int fmoe_abi_version(void);

/* ---- routing bookkeeping ------------------------------------------------ */

/* expert_count[e] += #{i : gate_idx[i] == e}; entries outside [0, n_expert)
 * (the -1 of dropped slots) are skipped.  The caller zero-fills.
 * Replaces fmoe_cuda_expert_count_impl, cuda/local_exchange.cuh:63-71
 * (bound as fmoe_cuda.expert_count, cuda/fmoe_cuda.cpp:119). */
int fmoe_expert_count(const int64_t *gate_idx, int32_t *expert_count,
                      int64_t n_slots, int64_t n_expert, void *stream);

/* Bytes of scratch the rank-based routing entry points below need. */
int64_t fmoe_routing_workspace_bytes(int64_t n_slots, int64_t n_expert);

/* Counting-sort placement.  cum_count enters as the int32 inclusive cumsum of
 * the expert counts and leaves as the exclusive one; pos[cum[e]-n_e .. cum[e])
 * receives the flat slot indices routed to expert e in DESCENDING index order
 * (what the reference kernel yields when its threads run one at a time in
 * ascending index).  pos holds n_pos entries; rows beyond it are not written.
 * Replaces fmoe_cuda_assign_pos_impl,
 * cuda/local_exchange.cuh:18-27 (fmoe_cuda.assign_pos, cuda/fmoe_cuda.cpp:120). */
int fmoe_assign_pos(int32_t *cum_count, const int64_t *gate, int64_t *pos,
                    int64_t n_pos, int64_t n_slots, int64_t n_expert,
                    void *workspace, int64_t workspace_bytes, void *stream);

/* One call for count + cumsum + placement (what fmoe/functions.py:19-42 does
 * with two kernels, a torch.cumsum and a host read in between):
 *   expert_count [n_expert] int64  <- histogram (overwritten, not accumulated)
 *   pos          [n_slots]  int64  <- first sum(expert_count) entries as in
 *                                     fmoe_assign_pos, the rest -1
 *   slot_to_row  [n_slots]  int64  <- inverse of pos: row of each slot in the
 *                                     expert-sorted order, -1 for dropped slots
 *                                     (may be NULL) */
int fmoe_route(const int64_t *gate, int64_t n_slots, int64_t n_expert,
               int64_t *expert_count, int64_t *pos, int64_t *slot_to_row,
               void *workspace, int64_t workspace_bytes, void *stream);

/* fmoe_route for callers that must not allocate (code under HIP graph capture,
 * serving loops, harnesses that forbid hipMalloc): same inputs, outputs and
 * results as fmoe_route, but the scratch is a fixed array of
 * FMOE_ROUTE_STATIC_SCRATCH_BYTES inside the library (one copy per GPU, held
 * until the process ends) instead of a caller's workspace, and the call makes
 * no hipMalloc / hipFree.  Sizes with
 * fmoe_routing_workspace_bytes(n_slots, n_expert) above that limit return
 * FMOE_ELIMIT.  All calls on one GPU share the array: calls that overlap in
 * time on one GPU (different streams or host threads) race.  The first call on
 * a device looks up the array's device address (hipGetSymbolAddress); make it
 * outside any stream capture.  No counterpart in the reference. */
#define FMOE_ROUTE_STATIC_SCRATCH_BYTES (1 << 20)
int fmoe_route_static(const int64_t *gate, int64_t n_slots, int64_t n_expert,
                      int64_t *expert_count, int64_t *pos,
                      int64_t *slot_to_row, void *stream);

/* The gate's top-k, its scores and the routing of fmoe_route in one call: per
 * token the top_k largest of n_expert logits (ties to the lower expert index,
 * choices in descending order of the logit),
 *   topk_idx   [n_tokens, top_k] int64
 *   topk_score [n_tokens, top_k] (dtype)  score_mode 0: the selected logits
 *              (what NaiveGate returns, fmoe/gates/naive_gate.py:32-42);
 *              1: softmax over the top_k selected logits
 * and, from the per-workgroup histograms the same pass leaves behind,
 * expert_count / pos / slot_to_row exactly as fmoe_route(topk_idx) gives them.
 * logits [n_tokens, n_expert] in FMOE_F32 / FMOE_BF16 / FMOE_F16; top_k 1, 2, 4
 * or 8 (FMOE_ELIMIT otherwise: use torch.topk and fmoe_route).  workspace: fmoe_routing_workspace_bytes(n_tokens*top_k, n_expert).
 * Replaces torch.topk (+ softmax) of fmoe/gates/naive_gate.py:26-42 followed by
 * count_by_gate, fmoe/functions.py:19-42. */
int fmoe_gate_topk_route(const void *logits, int64_t n_tokens, int64_t n_expert,
                         int64_t top_k, int dtype, int score_mode,
                         int64_t *topk_idx, void *topk_score,
                         int64_t *expert_count, int64_t *pos,
                         int64_t *slot_to_row, void *workspace,
                         int64_t workspace_bytes, void *stream);

/* The gate's linear layer folded into the same call, for small expert counts:
 * logits = x . w^T + bias are formed on chip (rounded to the element type as the
 * layer's output would be) and never written to memory; top-k, scores and
 * routing as above.  x [n_tokens, d_model], w [n_expert, d_model], bias
 * [n_expert] or NULL, all of `dtype`; x and w 16-byte aligned.
 * fmoe_gate_linear_supported says whether the shape is taken (at most 64
 * experts, top_k 1, 2, 4 or 8, d_model a whole number of 16-byte chunks);
 * FMOE_ELIMIT otherwise.  Replaces nn.Linear + torch.topk (+ softmax) of
 * fmoe/gates/naive_gate.py:26-42 followed by count_by_gate,
 * fmoe/functions.py:19-42.  Its backward is fmoe_gate_topk_backward followed by
 * the linear layer's own (two skinny library GEMMs). */
int fmoe_gate_linear_supported(int64_t d_model, int64_t n_expert, int64_t top_k,
                               int dtype);
int fmoe_gate_linear_topk_route(const void *x, const void *w, const void *bias,
                                int64_t n_tokens, int64_t d_model,
                                int64_t n_expert, int64_t top_k, int dtype,
                                int score_mode, int64_t *topk_idx,
                                void *topk_score, int64_t *expert_count,
                                int64_t *pos, int64_t *slot_to_row,
                                void *workspace, int64_t workspace_bytes,
                                void *stream);

/* Gradient of topk_score with respect to the logits, [n_tokens, n_expert]
 * (zero at experts that were not selected); score is only read in score_mode 1.
 * Replaces autograd's backward of torch.topk / softmax in the gate. */
int fmoe_gate_topk_backward(const void *grad_score, const void *score,
                            const int64_t *topk_idx, void *grad_logits,
                            int64_t n_tokens, int64_t n_expert, int64_t top_k,
                            int dtype, int score_mode, void *stream);

/* Noisy top-k gating in training mode (Shazeer et al. 2017; the behaviour of
 * fmoe/gates/noisy_gate.py:113-144) after the two linear products, in one
 * pass: with std = softplus(raw) + eps and noisy = clean + noise * std (clean,
 * raw, noise [n_tokens, n_expert] of `dtype`; noise is the caller's N(0,1)
 * draw), per token the top_k + 1 largest noisy logits,
 *   topk_idx [n_tokens, top_k] int64, gates [n_tokens, top_k] = softmax over
 *   the top_k largest;  thr_val / thr_idx [n_tokens, 2]: the top_k-th and
 *   (top_k+1)-th largest noisy logit and their experts (kept for the backward);
 *   load_partial [ceil(n_tokens*top_k / 2048), n_expert] float: per workgroup
 *   the sums over its tokens of Phi((clean - threshold) / std), threshold =
 *   the (top_k+1)-th largest noisy logit for an expert among the top_k, the
 *   top_k-th otherwise; the load is the sum of the rows;
 * and expert_count / pos / slot_to_row as fmoe_route(topk_idx) gives them.
 * top_k 1, 2, 4 or 8 and below n_expert <= 2048 (FMOE_ELIMIT otherwise).
 * workspace: fmoe_routing_workspace_bytes(n_tokens*top_k, n_expert). */
int fmoe_noisy_gate_forward(const void *clean, const void *raw,
                            const void *noise, double eps, int64_t n_tokens,
                            int64_t n_expert, int64_t top_k, int dtype,
                            int64_t *topk_idx, void *gates, float *thr_val,
                            int32_t *thr_idx, float *load_partial,
                            int64_t *expert_count, int64_t *pos,
                            int64_t *slot_to_row, void *workspace,
                            int64_t workspace_bytes, void *stream);

/* Its backward: from grad_gates [n_tokens, top_k] (`dtype`) and grad_load
 * [n_expert] (float), the gradients of the two logit matrices, grad_clean and
 * grad_raw [n_tokens, n_expert] (`dtype`), through the softmax, the smooth load
 * (including its thresholds) and the softplus.  Replaces autograd's backward of
 * fmoe/gates/noisy_gate.py:47-90,113-144. */
int fmoe_noisy_gate_backward(const void *clean, const void *raw,
                             const void *noise, double eps, int64_t n_tokens,
                             int64_t n_expert, int64_t top_k, int dtype,
                             const int64_t *topk_idx, const void *gates,
                             const float *thr_val, const int32_t *thr_idx,
                             const void *grad_gates, const float *grad_load,
                             void *grad_clean, void *grad_raw, void *stream);

/* ---- capacity balancing ------------------------------------------------- */

/* eca[w,e] = share of cap[e] granted to worker w, workers served in ascending
 * order; cap[e] is decremented by every proposal.  Replaces
 * fmoe_cuda_limit_by_capacity_impl, cuda/balancing.cuh:23-31
 * (fmoe_cuda.limit_by_capacity, cuda/fmoe_cuda.cpp:125). */
int fmoe_limit_by_capacity(const int64_t *ec, int32_t *cap, int64_t *eca,
                           int64_t n_expert, int64_t n_worker, void *stream);

/* new_gate_idx[i] = gate_idx[i] if fewer than ec[gate_idx[i]] slots with a
 * lower flat index chose the same expert, else -1.  ec[e] is decremented once
 * per slot that names e.  Slots already -1 stay -1.  Replaces
 * fmoe_cuda_prune_gate_by_capacity_impl, cuda/balancing.cuh:48-58
 * (fmoe_cuda.prune_gate_by_capacity, cuda/fmoe_cuda.cpp:126). */
int fmoe_prune_gate_by_capacity(const int64_t *gate_idx, int64_t *new_gate_idx,
                                int32_t *ec, int64_t n_slots, int64_t n_expert,
                                void *workspace, int64_t workspace_bytes,
                                void *stream);

/* ---- local scatter / gather (row permutes) ------------------------------ */

/* out[r,:] = index[r] >= 0 ? inp[index[r],:] : 0   for r in [0, n_out).
 * Replaces _local_scatter = torch.index_select, fmoe/functions.py:72-74. */
int fmoe_gather_rows(const void *inp, const int64_t *index, void *out,
                     int64_t n_out, int64_t n_inp, int64_t row_elems, int dtype,
                     void *stream);

/* out[r,:] = index[r] >= 0 ? inp[index[r] / index_div,:] : 0: the local scatter
 * of fmoe/functions.py:72-74 taken straight from the slot positions
 * (index = pos, index_div = top_k), without materialising pos // top_k
 * (fmoe/layers.py:133).  With the -1 entries that fmoe_route leaves past the
 * last routed slot, it can be launched over all n_slots entries of pos before
 * the host has read the expert counts. */
int fmoe_gather_rows_div(const void *inp, const int64_t *index,
                         int64_t index_div, void *out, int64_t n_out,
                         int64_t n_inp, int64_t row_elems, int dtype,
                         void *stream);

/* inverse[0..n_out) = -1, then inverse[pos[i]] = i for i in [0, n_pos).
 * With it, the zero-fill + index_copy_ of fmoe/functions.py:77-84
 * (maybe_overlap=False) is one fmoe_gather_rows(inp, inverse, out). */
int fmoe_invert_index(const int64_t *pos, int64_t n_pos, int64_t *inverse,
                      int64_t n_out, void *stream);

/* out[t,:] = sum_{j<top_k} rows inp[slot_to_row[t*top_k+j],:] (entries < 0
 * contribute nothing), summed in fp32 in ascending j.  The atomics-free form of
 * zeros().index_add_(pos // top_k), fmoe/functions.py:77-82, when the index is
 * known to be slot positions. */
int fmoe_reduce_slots(const void *inp, const int64_t *slot_to_row, void *out,
                      int64_t n_tokens, int64_t top_k, int64_t n_inp,
                      int64_t row_elems, int dtype, void *stream);

/* General out = zeros(n_out, row).index_add_(0, index, inp) with n_in source
 * rows (fmoe/functions.py:77-82, maybe_overlap=True), summed in fp32 in
 * ascending source row, so the result does not depend on scheduling.
 * workspace: fmoe_index_add_workspace_bytes(n_in, n_out). */
int64_t fmoe_index_add_workspace_bytes(int64_t n_in, int64_t n_out);
int fmoe_index_add_rows(const void *inp, const int64_t *index, void *out,
                        int64_t n_in, int64_t n_out, int64_t row_elems,
                        int dtype, void *workspace, int64_t workspace_bytes,
                        void *stream);

/* Masked tokens (FMoE's mask / mask_dict, fmoe/layers.py:288-319).  The kept
 * tokens are selected with fmoe_gather_rows over an index of the tokens whose
 * mask is 0 (fmoe_route with one "expert" yields that index and its inverse);
 * after the experts, the full token order is restored in one pass:
 *   out[t,:] = token_to_row[t] >= 0 ? src[token_to_row[t],:]
 *            : fill_row[t] >= 0    ? scale[t] * fill[fill_row[t],:]   (scale NULL: 1)
 *            : 0
 * src [n_src,row], fill [n_fill,row] (the mask_dict values), fill_row [n_tokens]
 * int64 (which mask_dict value a masked token takes, -1: none), scale
 * [n_tokens] (the sum of the token's gate scores when the combine is folded in).
 * Replaces the zeros() + boolean-index assignments of fmoe/layers.py:309-317. */
int fmoe_mask_restore(const void *src, const int64_t *token_to_row,
                      const void *scale, const void *fill,
                      const int64_t *fill_row, void *out, int64_t n_tokens,
                      int64_t n_src, int64_t n_fill, int64_t row_elems,
                      int dtype, void *stream);

/* Gradient of fmoe_mask_restore with respect to scale: grad_scale[t] =
 * <grad_out[t,:], fill[fill_row[t],:]> for masked tokens with a fill row, else
 * 0 (autograd of the bmm over the restored rows, fmoe/layers.py:321-322). */
int fmoe_mask_scale_grad(const void *grad_out, const int64_t *token_to_row,
                         const void *fill, const int64_t *fill_row,
                         void *grad_scale, int64_t n_tokens, int64_t n_fill,
                         int64_t row_elems, int dtype, void *stream);

/* ---- score-weighted combination of the top-k expert outputs ------------- */

/* out[t,:] = sum_{j<top_k} score[t,j] * x[t*top_k+j,:], accumulated in fp32.
 * x [n_tokens*top_k, row], score [n_tokens, top_k] (same dtype), out
 * [n_tokens, row].  Replaces torch.bmm(gate_score, x), fmoe/layers.py:321-322. */
int fmoe_combine_forward(const void *x, const void *score, void *out,
                         int64_t n_tokens, int64_t top_k, int64_t row_elems,
                         int dtype, void *stream);

/* Its backward: grad_x[t*top_k+j,:] = score[t,j] * grad_out[t,:] and
 * grad_score[t,j] = <grad_out[t,:], x[t*top_k+j,:]>. */
int fmoe_combine_backward(const void *grad_out, const void *x, const void *score,
                          void *grad_x, void *grad_score, int64_t n_tokens,
                          int64_t top_k, int64_t row_elems, int dtype,
                          void *stream);

/* The copy back to slot order folded into the combination:
 * out[t,:] = sum_j score[t,j] * rows[slot_to_row[t*top_k+j],:], where rows
 * [n_rows, row] are the experts' outputs in expert-sorted order and a
 * negative slot_to_row entry (dropped slot) contributes nothing.  One pass in
 * place of _local_gather in MOEGather.forward (fmoe/functions.py:77-84,
 * 285-312) followed by torch.bmm (fmoe/layers.py:321-322). */
int fmoe_gather_combine_forward(const void *rows, const int64_t *slot_to_row,
                                const void *score, void *out, int64_t n_tokens,
                                int64_t top_k, int64_t n_rows,
                                int64_t row_elems, int dtype, void *stream);

/* Its backward: grad_rows[slot_to_row[s],:] = score[s] * grad_out[s/top_k,:]
 * for every kept slot s, grad_score[t,j] = <grad_out[t,:], rows[...]> (0 for a
 * dropped slot).  Every row of grad_rows is written exactly once when
 * slot_to_row, restricted to the kept slots, is one-to-one onto [0, n_rows)
 * (as fmoe_route produces it); rows no slot maps to are left untouched. */
int fmoe_gather_combine_backward(const void *grad_out, const void *rows,
                                 const int64_t *slot_to_row, const void *score,
                                 void *grad_rows, void *grad_score,
                                 int64_t n_tokens, int64_t top_k,
                                 int64_t n_rows, int64_t row_elems, int dtype,
                                 void *stream);

/* ---- per-expert linear (one grouped GEMM over ragged row segments) ------ */

/* y[seg_e,:] = x[seg_e,:] . w[e]^T (+ bias[e]); seg_e are consecutive row
 * ranges of lengths expert_count_host[e].  x [S,in], w [E,out,in],
 * bias [E,out] or NULL, y [S,out].  Replaces fmoe_cuda_linear_forward_impl,
 * cuda/parallel_linear.cuh:55-88 (fmoe_cuda.linear_forward). */
int fmoe_linear_forward(const void *x, const void *w, const void *bias, void *y,
                        const int64_t *expert_count_host, int64_t n_expert,
                        int64_t in_feat, int64_t out_feat, int dtype,
                        void *stream);

/* grad_x[seg_e,:] = grad_y[seg_e,:] . w[e];  grad_w[e] = grad_y[seg_e]^T . x[seg_e]
 * (zeros for an empty expert);  grad_b[e] = column sums of grad_y[seg_e] when
 * grad_b != NULL.  Replaces fmoe_cuda_linear_backward_impl,
 * cuda/parallel_linear.cuh:90-161 (fmoe_cuda.linear_backward). */
int fmoe_linear_backward(const void *grad_y, const void *x, const void *w,
                         void *grad_x, void *grad_w, void *grad_b,
                         const int64_t *expert_count_host, int64_t n_expert,
                         int64_t in_feat, int64_t out_feat, int dtype,
                         void *stream);

/* The first linear of an expert MLP with its activation in the GEMM's epilogue:
 *   pre[seg_e] = x[seg_e] . w[e]^T + bias[e]   (stored when pre != NULL)
 *   y[seg_e]   = act(pre[seg_e])
 * Replaces FMoELinear followed by the activation module as two kernels,
 * fmoe/transformer.py:22-30 (_Expert.forward: htoh4, activation). */
int fmoe_linear_act_forward(const void *x, const void *w, const void *bias,
                            void *pre, void *y,
                            const int64_t *expert_count_host, int64_t n_expert,
                            int64_t in_feat, int64_t out_feat, int dtype,
                            int activation, void *stream);

/* Data gradient of the second linear with the activation's derivative in the
 * epilogue: grad_x[seg_e] = (grad_y[seg_e] . w[e]) * act'(pre[seg_e]), i.e. the
 * gradient with respect to the first linear's pre-activation.  w is
 * [E, out_feat, in_feat], pre and grad_x are [rows, in_feat].  For ReLU the
 * post-activation may be passed as pre (same sign pattern).  Replaces the
 * data-grad half of fmoe_cuda_linear_backward_impl,
 * cuda/parallel_linear.cuh:122-132, followed by torch's activation backward
 * (autograd of fmoe/transformer.py:22-30). */
int fmoe_linear_dact_backward(const void *grad_y, const void *w, const void *pre,
                              void *grad_x, const int64_t *expert_count_host,
                              int64_t n_expert, int64_t in_feat,
                              int64_t out_feat, int dtype, int activation,
                              void *stream);

/* ---- the same products without the expert counts on the host ------------ */

/* The four entry points above read expert_count_host on the host, as
 * cuda/parallel_linear.cuh:69,85,113 does, so a layer call has to wait for a
 * device-to-host copy of the counts between its routing kernels and its first
 * GEMM.  The entry points below take the row segments from a table in DEVICE
 * memory instead, which one small kernel builds from the counts fmoe_route /
 * fmoe_gate_topk_route leave on the device; nothing waits for the host and the
 * whole layer can be captured in a HIP graph.  No counterpart in the reference
 * (what they replace: the host loops of cuda/parallel_linear.cuh:55-161 and the
 * .item() / .cpu() reads of fmoe/functions.py:38-40,64-68).
 *
 * Bytes of a table for at most rows_cap expert-sorted rows over n_expert experts. */
int64_t fmoe_segment_table_bytes(int64_t rows_cap, int64_t n_expert);

/* Builds the table from expert_count [n_expert] int64 (device).  Counts are
 * taken in order and clamped so that they never add up to more than rows_cap
 * (a count < 0 reads as 0).  segment_table: 16-byte aligned device memory of
 * fmoe_segment_table_bytes(rows_cap, n_expert) bytes. */
int fmoe_segment_table_build(const int64_t *expert_count, int64_t n_expert,
                             int64_t rows_cap, void *segment_table,
                             int64_t table_bytes, void *stream);

/* 1 when the three entry points below take this shape (16- or 32-bit floats,
 * feature sizes that are multiples of 16 bytes), else 0.  Host only. */
int fmoe_linear_dev_supported(int64_t in_feat, int64_t out_feat, int dtype);

/* Bytes of workspace with which the two row-ragged products below can split a
 * last, partial round of tiles along the contraction (the host-count entry
 * points keep such a workspace inside the library; here it is the caller's, so
 * that nothing on this path allocates); 0 when a contraction of `contraction`
 * elements is too short to be split at all.  workspace may always be NULL: the
 * last round is then not split. */
int64_t fmoe_linear_dev_workspace_bytes(int64_t contraction, int dtype);

/* fmoe_linear_forward / fmoe_linear_act_forward over a device table:
 *   pre[seg_e] = x[seg_e] . w[e]^T + bias[e]  (stored when pre != NULL)
 *   y[seg_e]   = act(pre[seg_e])              (activation FMOE_ACT_NONE: y = pre)
 * x, pre, y have at least rows_cap rows, of which the table's rows are touched.
 * x_row_index != NULL: expert-sorted row r is read from row
 * x_row_index[r] / x_index_div of x [x_total_rows, in_feat] instead of row r --
 * the local scatter (_local_scatter, fmoe/functions.py:72-74) done by the
 * GEMM's loader, with x_row_index = pos and x_index_div = top_k; x must then
 * be smaller than 2 GiB. */
int fmoe_linear_forward_dev(const void *x, const int64_t *x_row_index,
                            int64_t x_index_div, int64_t x_total_rows,
                            const void *w, const void *bias, void *pre, void *y,
                            const void *segment_table, int64_t n_expert,
                            int64_t rows_cap, int64_t in_feat, int64_t out_feat,
                            int dtype, int activation, void *workspace,
                            int64_t workspace_bytes, void *stream);

/* Data gradient, as fmoe_linear_dact_backward (activation FMOE_ACT_NONE: the
 * plain data gradient of fmoe_linear_backward, pre ignored). */
int fmoe_linear_dgrad_dev(const void *grad_y, const void *w, const void *pre,
                          void *grad_x, const void *segment_table,
                          int64_t n_expert, int64_t rows_cap, int64_t in_feat,
                          int64_t out_feat, int dtype, int activation,
                          void *workspace, int64_t workspace_bytes,
                          void *stream);

/* Weight and bias gradient, as the grad_w / grad_b half of fmoe_linear_backward
 * (an expert without rows gets zeros; grad_b may be NULL). */
int fmoe_linear_wgrad_dev(const void *grad_y, const void *x, void *grad_w,
                          void *grad_b, const void *segment_table,
                          int64_t n_expert, int64_t rows_cap, int64_t in_feat,
                          int64_t out_feat, int dtype, void *stream);

/* How a forward / data-grad launch of `total_tiles` output tiles (256 x 256, or
 * 128 x 256 / 128 x 128 for small launches) of a 16-bit element type with
 * `contraction_slabs` slabs of 128 contraction bytes (fp32 launches count
 * every slab twice in the plan's thresholds: half the elements at a quarter
 * of the rate) is spread over `compute_units` (0: the current device's):
 * plan_host[0] tiles are computed whole, one workgroup each; the rest -- the
 * last, partial round of the chip when it fills at most half of it -- are
 * split along the contraction into plan_host[1] parts of plan_host[2] slabs,
 * whose fp32 partial sums are added in ascending order before the epilogue.
 * Host only.  No counterpart in the reference (its per-expert cuBLAS calls,
 * cuda/parallel_linear.cuh:55-88, leave this to the library). */
int fmoe_gemm_tail_plan(int64_t total_tiles, int64_t contraction_slabs,
                        int compute_units, int64_t *plan_host);

/* ---- fused expert MLP, chunked pipeline at world_size 1 ----------------- */

typedef struct fmoe_mlp_params {
    const void *w1;   /* [E, d_hidden, d_model] */
    const void *b1;   /* [E, d_hidden] or NULL  */
    const void *w2;   /* [E, d_model, d_hidden] */
    const void *b2;   /* [E, d_model] or NULL   */
    int64_t n_expert, d_model, d_hidden;
    int dtype;        /* FMOE_F32 / FMOE_BF16 / FMOE_F16 */
    int activation;   /* FMOE_ACT_* */
} fmoe_mlp_params;

/* Row bounds of the pipeline's chunks: chunk c covers the expert-sorted rows
 * [bounds_host[c], bounds_host[c+1]), bounds_host has n_chunks + 1 entries.
 * Every bound lies on a row-tile edge of the grouped GEMM (256 rows, counted
 * from each expert's first row), and when the chunks are long enough all but
 * the last hold a tile count whose launches, for output widths d_model and
 * d_hidden, are whole rounds of `compute_units` workgroups (0: the current
 * device's count, 256 without a device).  n_chunks == 0 asks for the library's
 * own choice, as in the two calls below: up to 4 chunks, but only as many as
 * leave every chunk four rounds of tiles in its narrower product; bounds_host
 * then has 5 entries, those beyond the chosen count repeat the end.  Host
 * only, no GPU work.  Plays the part of the worker-group stepping of
 * cuda/fused_compute.cuh:276-280. */
int fmoe_fused_chunk_bounds(const int64_t *expert_count_host, int64_t n_expert,
                            int n_chunks, int64_t d_model, int64_t d_hidden,
                            int compute_units, int64_t *bounds_host);

/* 1 when fmoe_fused_mlp_forward can take buf_in = NULL for this layer and input
 * (MFMA path: 16-byte aligned pointers, feature sizes that are multiples of 16
 * bytes; token matrix below 2 GiB), else 0.  Host only. */
int fmoe_fused_scatter_in_loader(const fmoe_mlp_params *p, const void *inp,
                                 int64_t n_tokens);

/* Forward of scatter -> Linear -> act -> Linear -> gather over `n_chunks`
 * contiguous chunks of the expert-sorted rows, chunk c+1's scatter and chunk
 * c-1's gather running beside chunk c's GEMMs on the library's own streams,
 * chained by events to `stream` (fork at entry, join at exit).  n_chunks == 0:
 * the library chooses (see fmoe_fused_chunk_bounds); with a single chunk all
 * work is enqueued on `stream` itself and no event is used.
 *   inp        [n_tokens, d_model]
 *   pos        [n_rows] int64   flat slot of every expert-sorted row
 *   slot_to_row[n_tokens*top_k] int64 (inverse of pos, -1 = dropped)
 *   buf_in     [n_rows, d_model]   scattered input  (kept for backward); NULL: the
 *              first GEMM reads the token rows through pos in its loader and no
 *              sorted copy of the input is made (only where
 *              fmoe_fused_scatter_in_loader says so)
 *   buf_pre    [n_rows, d_hidden]  pre-activation   (kept for backward)
 *   buf_mid    [n_rows, d_hidden]  post-activation  (kept for backward)
 *   buf_out    [n_rows, d_model]   expert output
 *   out        [n_tokens*top_k, d_model]  zero rows for dropped slots; NULL:
 *              the copy to slot order is skipped and the caller reads buf_out
 *              (e.g. with fmoe_gather_combine_forward)
 * Replaces fmoe_cuda_fused_forward_impl at one worker,
 * cuda/fused_compute.cuh:250-388 (fmoe_cuda.fused_forward) together with the
 * _local_scatter/_local_gather around it, fmoe/fused_functions.py:22-32. */
int fmoe_fused_mlp_forward(const fmoe_mlp_params *p, const void *inp,
                           const int64_t *pos, const int64_t *slot_to_row,
                           const int64_t *expert_count_host, int64_t n_tokens,
                           int64_t top_k, int64_t n_rows, void *buf_in,
                           void *buf_pre, void *buf_mid, void *buf_out,
                           void *out, int n_chunks, void *stream);

/* Backward of the same pipeline.  grad_out [n_tokens*top_k, d_model]; NULL: the
 * caller has already put the gradient rows in expert-sorted order into g_out
 * (e.g. with fmoe_gather_combine_backward).  inp != NULL: the forward kept no
 * sorted copy of the input (buf_in = NULL there); buf_in is then scratch that
 * this call fills from inp [n_tokens, d_model] on its permute lane.
 * Scratch (caller-allocated): g_out [n_rows,d_model], g_mid [n_rows,d_hidden],
 * g_in [n_rows,d_model].  Results: grad_inp [n_tokens,d_model], grad_w1/2,
 * grad_b1/2 (bias grads may be NULL).  The data gradients run chunk by chunk;
 * the weight gradients run once over all rows after the last chunk, so an
 * expert's gradient is rounded once however the rows are chunked (the
 * reference accumulates them step by step, cuda/fused_compute.cuh:123).
 * Replaces fmoe_cuda_fused_backward_impl at one worker,
 * cuda/fused_compute.cuh:391-542 (fmoe_cuda.fused_backward). */
int fmoe_fused_mlp_backward(const fmoe_mlp_params *p, const void *grad_out,
                            const int64_t *pos, const int64_t *slot_to_row,
                            const int64_t *expert_count_host, int64_t n_tokens,
                            int64_t top_k, int64_t n_rows, const void *inp,
                            void *buf_in, const void *buf_pre,
                            const void *buf_mid,
                            void *g_out, void *g_mid, void *g_in,
                            void *grad_inp, void *grad_w1, void *grad_b1,
                            void *grad_w2, void *grad_b2, int n_chunks,
                            void *stream);

/* ---- per-launch timing of the library's kernels (off by default) ------- */

/* Kernel classes, in the order of the arrays fmoe_profile_collect fills:
 * 0 grouped GEMM forward, 1 grouped GEMM data-grad, 2 grouped GEMM weight-grad
 * (work = flop); 3 bias grad, 4 gather rows, 5 scatter rows, 6 reduce slots,
 * 7 index add, 8 score combine (work = algorithmic bytes).  No counterpart in the reference
 * (its cuda/utils/timer.hh is commented out); used by bench.py to time each
 * kernel with HIP events on the stream it is launched on. */
int fmoe_profile_enable(int on);
int fmoe_profile_classes(void);
/* Synchronises the device, then returns per class the launches recorded since
 * the last collect, their summed duration (ms) and summed work. */
int fmoe_profile_collect(int64_t *launches, double *milliseconds, double *work,
                         int n_classes);

#ifdef __cplusplus
}
#endif
#endif /* FMOE_HIP_H */
