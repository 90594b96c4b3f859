// Row-permute launchers shared between the C ABI (permute.hip) and the fused
// pipeline (pipeline.hip).
#pragma once
#include "common.hpp"

namespace fmoe {

// out[r,:] = inp[index[r] / divisor,:] for r in [0, n_out); rows whose index is
// negative or whose source is outside [0, n_inp) become zero.
int permute_gather_rows(const void *inp, const int64_t *index, int64_t divisor, void *out, int64_t n_out,
                        int64_t n_inp, int64_t row_elems, int dtype, hipStream_t stream);

// out[index[r],:] = inp[r,:] for r in [0, n_in); targets outside [0, n_out) are skipped.
int permute_scatter_rows(const void *inp, const int64_t *index, void *out, int64_t n_in, int64_t n_out,
                         int64_t row_elems, int dtype, hipStream_t stream);

// out[r,:] = 0 for every r in [0, n_out) with index[r] < 0.
int permute_zero_unmapped(const int64_t *index, void *out, int64_t n_out, int64_t row_elems, int dtype,
                          hipStream_t stream);

}  // namespace fmoe
