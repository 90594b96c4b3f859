// Grouped GEMM over ragged expert segments (gfx950): host-side interface shared
// by the per-expert linear entry points and the fused MLP pipeline.
#pragma once
#include "common.hpp"

namespace fmoe {

// What the epilogue does with the fp32 accumulator tile.
enum Epilogue {
    kEpiStore = 0,    // C = acc (+ bias[col])
    kEpiBiasAct = 1,  // pre = acc + bias[col]; aux = pre (if aux); C = act(pre)
    kEpiDAct = 2,     // C = acc * act'(aux)          (aux = saved pre-activation)
};

constexpr int kMaxGroupExperts = 256;  // experts per launch (table lives in kernel arguments)

// Row segments of the experts covered by one launch.  seg[i] .. seg[i+1] are the
// rows of expert first_expert + i; for a chunk of the fused pipeline the rows
// are already clipped to the chunk.
struct SegmentTable {
    int32_t n;                            // experts in this launch
    int32_t first_expert;                 // global index of seg[0]'s expert
    int32_t seg[kMaxGroupExperts + 1];    // row offsets
    int32_t tile[kMaxGroupExperts + 1];   // prefix of row tiles (ragged-M launches)
};

// Segment table in device memory, for launches that must not wait for the expert counts to
// reach the host: built by segment_table_kernel from the routing's counts, read by the grouped
// GEMM through scalar loads.  All entries are int32:
//   [0] n_expert   [1] rows (sum of the counts)   [2] row tiles of 256   [3] row tiles of 128
//   [4] offset of the 256-row tile map            [5] offset of the 128-row tile map
//   [6] rows_cap the table was laid out for       [7] 0
//   [8 .. 8+E]           seg: first row of every expert, seg[E] = rows
//   [.. +E+1] [.. +E+1]  exclusive prefix of the experts' row tiles, 256 and 128 rows high
//   tile maps            one {expert, first row, rows, 0} per row tile, 16-byte aligned
// A launch is sized for the most row tiles `rows_cap` rows can make (rows_cap / BM + E); the
// workgroups beyond the table's tile count leave at once.
namespace segtab {
constexpr int kHeader = 8;
constexpr int kRows = 1, kTiles256 = 2, kTiles128 = 3, kMap256 = 4, kMap128 = 5, kRowsCap = 6;
__host__ __device__ inline int64_t cap_tiles(int64_t rows_cap, int64_t n_expert, int block_rows) {
    return rows_cap / block_rows + (n_expert < rows_cap ? n_expert : rows_cap);
}
__host__ __device__ inline int64_t seg_off() { return kHeader; }
__host__ __device__ inline int64_t pfx256_off(int64_t n_expert) { return kHeader + (n_expert + 1); }
__host__ __device__ inline int64_t pfx128_off(int64_t n_expert) { return kHeader + 2 * (n_expert + 1); }
__host__ __device__ inline int64_t map256_off(int64_t n_expert) { return (kHeader + 3 * (n_expert + 1) + 3) / 4 * 4; }
__host__ __device__ inline int64_t map128_off(int64_t rows_cap, int64_t n_expert) {
    return map256_off(n_expert) + 4 * cap_tiles(rows_cap, n_expert, 256);
}
__host__ __device__ inline int64_t total_ints(int64_t rows_cap, int64_t n_expert) {
    return map128_off(rows_cap, n_expert) + 4 * cap_tiles(rows_cap, n_expert, 128);
}
}  // namespace segtab

struct LinearForwardArgs {
    const void *x;      // [rows, in]; with x_row_index: the token matrix [x_total_rows, in]
    const void *w;      // [E, out, in]
    const void *bias;   // [E, out] or null
    void *y;            // [rows, out]
    void *aux;          // [rows, out] pre-activation copy (kEpiBiasAct) or null
    int64_t in_feat, out_feat;
    int dtype, epilogue, activation;
    // optional: sorted row r is read from row x_row_index[r] / x_index_div of x (local scatter in the
    // loader); only honoured where linear_forward_can_gather() says so
    const int64_t *x_row_index = nullptr;
    int64_t x_index_div = 1, x_total_rows = 0;
    // optional: the segments come from a device table (segtab) laid out for dev_rows_cap rows; the
    // host counts are then not read (may be NULL) and the row range must be everything
    const int32_t *dev_tab = nullptr;
    int64_t dev_rows_cap = 0;
    // optional, with dev_tab: workspace of linear_dev_workspace_bytes() for the split of a last, partial
    // round of tiles (without it such a round is not split)
    void *dev_workspace = nullptr;
    int64_t dev_workspace_bytes = 0;
};

// Bytes of workspace with which a launch over a device table can split its last round of tiles along a
// contraction of `contraction` elements; 0 when a contraction this short is never split.
int64_t linear_dev_workspace_bytes(int64_t contraction, int dtype);

// Whether the forward product can read its rows through an index: the MFMA path (aligned pointers,
// feature sizes that are multiples of 16 bytes) and a token matrix of less than 2 GiB.
bool linear_forward_can_gather(const LinearForwardArgs &a);

struct LinearDgradArgs {
    const void *gy;     // [rows, out]
    const void *w;      // [E, out, in]
    void *gx;           // [rows, in]
    const void *aux;    // [rows, in] pre-activation (kEpiDAct) or null
    int64_t in_feat, out_feat;
    int dtype, epilogue, activation;
    const int32_t *dev_tab = nullptr;  // as in LinearForwardArgs
    int64_t dev_rows_cap = 0;
    void *dev_workspace = nullptr;
    int64_t dev_workspace_bytes = 0;
};

struct LinearWgradArgs {
    const void *gy;     // [rows, out]
    const void *x;      // [rows, in]
    void *gw;           // [E, out, in]
    void *gb;           // [E, out] bias gradient (column sums of gy per expert) or null
    int64_t in_feat, out_feat;
    int dtype;
    const int32_t *dev_tab = nullptr;  // as in LinearForwardArgs
    int64_t dev_rows_cap = 0;
};

// counts[e] rows for experts [0, n_expert), restricted to rows [row_lo, row_hi)
// of the expert-sorted order.  Launches on `stream`; for more than
// kMaxGroupExperts experts the work is split into several launches.
int grouped_linear_forward(const LinearForwardArgs &a, const int64_t *counts_host, int64_t n_expert,
                           int64_t row_lo, int64_t row_hi, hipStream_t stream);
int grouped_linear_dgrad(const LinearDgradArgs &a, const int64_t *counts_host, int64_t n_expert,
                         int64_t row_lo, int64_t row_hi, hipStream_t stream);
// Weight gradient over the rows [row_lo, row_hi).  An expert is written by the
// chunk that holds any of its rows; an expert without rows is zero-filled by
// the chunk that contains its (empty) position, the last chunk taking the
// position row_hi.  An expert whose rows began before row_lo adds to what the
// earlier chunk left (cuda/fused_compute.cuh:123, beta_weight).
int grouped_linear_wgrad(const LinearWgradArgs &a, const int64_t *counts_host, int64_t n_expert,
                         int64_t row_lo, int64_t row_hi, bool last_chunk, hipStream_t stream);
// grad_b[e, c] = column sums of gy over the rows of expert e; same chunk rules.
int grouped_bias_grad(const void *gy, void *gb, int64_t out_feat, int dtype, const int64_t *counts_host,
                      int64_t n_expert, int64_t row_lo, int64_t row_hi, bool last_chunk, hipStream_t stream);

}  // namespace fmoe
