// Fused expert-MLP pipeline for one worker (gfx950).
//
// The expert-sorted rows are cut into `n_chunks` contiguous chunks.  Three HIP
// streams owned by the library run, for chunk c,
//     permute-in  : gather token rows into the sorted buffer
//     compute     : grouped GEMM 1 (+bias, activation), grouped GEMM 2 (+bias)
//     permute-out : write expert outputs back to slot order
// so that chunk c+1's permute-in and chunk c-1's permute-out overlap chunk c's
// GEMMs.  Chunks are chained by events (in_ready[c], out_ready[c]); the
// caller's stream forks into the three streams at entry and joins them at
// exit, so the call behaves like one asynchronous operation on that stream.
// Backward mirrors this: gather grad rows, dgrad/wgrad of both linears with the
// activation derivative folded into the first dgrad's epilogue, and a final
// per-token reduction of the k expert-row gradients.  A caller that combines the
// experts' outputs straight from the sorted buffer passes out = NULL (no
// permute-out stage), and grad_out = NULL in the backward when it has already
// written the gradient rows in sorted order (no permute-in stage).
//
// All streams use the default priority.  Streams and events are created once per
// device and reused; host threads that call the fused entry points on the same
// device are serialised by a per-device mutex while they enqueue.
#include "grouped_gemm.hpp"
#include "permute.hpp"

#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <vector>

namespace fmoe {
namespace {

constexpr int kMaxChunks = 32;

struct DeviceLanes {
    bool ready = false;
    hipStream_t in = nullptr, compute = nullptr, out = nullptr;
    hipEvent_t fork = nullptr, join_in = nullptr, join_compute = nullptr, join_out = nullptr, regather = nullptr;
    hipEvent_t in_ready[kMaxChunks] = {};
    hipEvent_t out_ready[kMaxChunks] = {};
};

std::mutex g_lanes_mutex;
DeviceLanes g_lanes[16];
// One fused call at a time enqueues on a device's lanes: host threads that call the fused entry points
// on the same device are serialised here (their work is still ordered by their own streams' fork/join).
std::mutex g_enqueue_mutex[16];

int get_lanes(DeviceLanes **out) {
    int dev = 0;
    FMOE_HIP_CHECK(hipGetDevice(&dev));
    FMOE_REQUIRE(dev >= 0 && dev < 16, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_lanes_mutex);
    DeviceLanes &l = g_lanes[dev];
    if (!l.ready) {
        FMOE_HIP_CHECK(hipStreamCreateWithFlags(&l.in, hipStreamNonBlocking));
        FMOE_HIP_CHECK(hipStreamCreateWithFlags(&l.compute, hipStreamNonBlocking));
        FMOE_HIP_CHECK(hipStreamCreateWithFlags(&l.out, hipStreamNonBlocking));
        hipEvent_t *single[] = {&l.fork, &l.join_in, &l.join_compute, &l.join_out, &l.regather};
        for (hipEvent_t *e : single) FMOE_HIP_CHECK(hipEventCreateWithFlags(e, hipEventDisableTiming));
        for (int c = 0; c < kMaxChunks; ++c) {
            FMOE_HIP_CHECK(hipEventCreateWithFlags(&l.in_ready[c], hipEventDisableTiming));
            FMOE_HIP_CHECK(hipEventCreateWithFlags(&l.out_ready[c], hipEventDisableTiming));
        }
        l.ready = true;
    }
    *out = &l;
    return FMOE_OK;
}

// The streams a call enqueues on: the library's three lanes, or -- with a single chunk, where
// nothing can overlap -- the caller's own stream for everything, with no events at all.
struct CallStreams {
    hipStream_t in, compute, out;
    bool lanes;  // false: all three are the caller's stream
};
inline int record(const CallStreams &cs, hipEvent_t ev, hipStream_t s) {
    if (cs.lanes) FMOE_HIP_CHECK(hipEventRecord(ev, s));
    return FMOE_OK;
}
inline int wait(const CallStreams &cs, hipStream_t s, hipEvent_t ev) {
    if (cs.lanes) FMOE_HIP_CHECK(hipStreamWaitEvent(s, ev, 0));
    return FMOE_OK;
}

int fork_lanes(DeviceLanes *l, hipStream_t caller) {
    FMOE_HIP_CHECK(hipEventRecord(l->fork, caller));
    FMOE_HIP_CHECK(hipStreamWaitEvent(l->in, l->fork, 0));
    FMOE_HIP_CHECK(hipStreamWaitEvent(l->compute, l->fork, 0));
    FMOE_HIP_CHECK(hipStreamWaitEvent(l->out, l->fork, 0));
    return FMOE_OK;
}

int join_lanes(DeviceLanes *l, hipStream_t caller) {
    FMOE_HIP_CHECK(hipEventRecord(l->join_in, l->in));
    FMOE_HIP_CHECK(hipEventRecord(l->join_compute, l->compute));
    FMOE_HIP_CHECK(hipEventRecord(l->join_out, l->out));
    FMOE_HIP_CHECK(hipStreamWaitEvent(caller, l->join_in, 0));
    FMOE_HIP_CHECK(hipStreamWaitEvent(caller, l->join_compute, 0));
    FMOE_HIP_CHECK(hipStreamWaitEvent(caller, l->join_out, 0));
    return FMOE_OK;
}

int check_common(const char *who, const fmoe_mlp_params *p, const int64_t *counts, int64_t n_tokens,
                 int64_t top_k, int64_t n_rows, int n_chunks) {
    FMOE_REQUIRE(p != nullptr, "%s: params is NULL", who);
    FMOE_REQUIRE(p->dtype == FMOE_F32 || p->dtype == FMOE_BF16 || p->dtype == FMOE_F16,
                 "%s: dtype %d not supported by the fused path (f32, bf16, f16)", who, p->dtype);
    FMOE_REQUIRE(p->activation >= FMOE_ACT_NONE && p->activation <= FMOE_ACT_GELU, "%s: activation %d", who,
                 p->activation);
    FMOE_REQUIRE(p->n_expert >= 1 && p->d_model >= 1 && p->d_hidden >= 1, "%s: bad sizes", who);
    FMOE_REQUIRE(p->w1 && p->w2, "%s: NULL weights", who);
    FMOE_REQUIRE(n_tokens >= 0 && top_k >= 1 && n_rows >= 0 && n_rows <= n_tokens * top_k,
                 "%s: n_tokens=%lld top_k=%lld n_rows=%lld", who, (long long)n_tokens, (long long)top_k,
                 (long long)n_rows);
    FMOE_REQUIRE(n_chunks >= 0 && n_chunks <= kMaxChunks, "%s: n_chunks=%d (0 = chosen by the library, 1..%d)", who,
                 n_chunks, kMaxChunks);
    FMOE_REQUIRE(counts != nullptr, "%s: expert_count_host is NULL", who);
    int64_t s = 0;
    for (int64_t e = 0; e < p->n_expert; ++e) {
        FMOE_REQUIRE(counts[e] >= 0, "%s: negative expert count", who);
        s += counts[e];
    }
    FMOE_REQUIRE(s == n_rows, "%s: expert counts sum to %lld, n_rows is %lld", who, (long long)s,
                 (long long)n_rows);
    return FMOE_OK;
}

constexpr int kTileRows = 256;  // row-tile height of the grouped GEMM (a 128-row launch tiles the same edges)

int64_t gcd64(int64_t a, int64_t b) { return b == 0 ? a : gcd64(b, a % b); }

// Row position at which the first `tiles` row tiles of the expert-sorted order end (an
// expert's rows are tiled from the expert's own first row, its last tile may be partial).
int64_t rows_of_tiles(const int64_t *counts, int64_t n_expert, int64_t tiles) {
    int64_t start = 0;
    for (int64_t e = 0; e < n_expert && tiles > 0; ++e) {
        const int64_t t = ceil_div(counts[e], kTileRows);
        if (tiles < t) return start + tiles * kTileRows;
        tiles -= t;
        start += counts[e];
    }
    return start;
}

// Chunk c covers the sorted rows [bounds[c], bounds[c+1]).  Every bound lies on the edge of a
// row tile of the grouped GEMM, so cutting an expert's rows adds no partial tile.  A chunk of
// t row tiles launches t * ceil(width / 256) workgroups per product, and the chip runs them
// `cus` at a time, a last partial round costing as much as a whole one: when the chunks are long
// enough, all but the last get a tile count that makes both products' launches (output widths
// d_model and d_hidden) whole numbers of rounds, and the last one takes what is left.
void chunk_bounds(const int64_t *counts, int64_t n_expert, int64_t n_rows, int n_chunks, int64_t d_model,
                  int64_t d_hidden, int cus, int64_t *bounds) {
    int64_t tiles = 0;
    for (int64_t e = 0; e < n_expert; ++e) tiles += ceil_div(counts[e], kTileRows);
    // smallest tile count whose launches fill whole rounds for both widths
    const int64_t wd = ceil_div(d_model, 256), wh = ceil_div(d_hidden, 256);
    const int64_t ud = cus / gcd64(cus, wd), uh = cus / gcd64(cus, wh);
    const int64_t unit = ud / gcd64(ud, uh) * uh;
    int64_t per = -1;  // row tiles of every chunk but the last; -1: split the tiles evenly
    if (unit * n_chunks <= tiles) {
        per = (tiles + (int64_t)n_chunks * unit / 2) / ((int64_t)n_chunks * unit) * unit;  // nearest multiple to tiles / n_chunks
        if (per * (n_chunks - 1) >= tiles) per -= unit;
    }
    bounds[0] = 0;
    for (int c = 1; c < n_chunks; ++c) {
        const int64_t t = per > 0 ? per * c : tiles * c / n_chunks;
        const int64_t b = rows_of_tiles(counts, n_expert, t);
        bounds[c] = b < bounds[c - 1] ? bounds[c - 1] : b;
    }
    bounds[n_chunks] = n_rows;
}

// Chunk count when the caller leaves it to the library (n_chunks == 0): up to kAutoChunks, but
// only as many as leave every chunk at least four rounds of tiles in its narrower product --
// shorter launches lose more to partly filled rounds than the overlapped permutes gain (measured:
// 16384 tokens x top-2, d 1024 / h 4096: 1 chunk 2.16 ms per step, 2 chunks 2.27, 4 chunks 2.73).
constexpr int kAutoChunks = 4;
int auto_chunks(const int64_t *counts, int64_t n_expert, int64_t d_model, int64_t d_hidden, int cus) {
    int64_t tiles = 0;
    for (int64_t e = 0; e < n_expert; ++e) tiles += ceil_div(counts[e], kTileRows);
    const int64_t narrow = std::min(ceil_div(d_model, 256), ceil_div(d_hidden, 256));
    const int64_t min_tiles = std::max<int64_t>(1, ceil_div((int64_t)4 * cus, narrow));
    return (int)std::max<int64_t>(1, std::min<int64_t>(kAutoChunks, tiles / min_tiles));
}

int compute_units_or_default() {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return 256; }
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return 256;
    }
    return n;
}

inline const char *at(const void *base, int64_t row, int64_t row_elems, int dtype) {
    return static_cast<const char *>(base) + row * row_elems * dtype_bytes(dtype);
}
inline char *at(void *base, int64_t row, int64_t row_elems, int dtype) {
    return static_cast<char *>(base) + row * row_elems * dtype_bytes(dtype);
}

}  // namespace
}  // namespace fmoe

using namespace fmoe;

extern "C" int fmoe_fused_chunk_bounds(const int64_t *expert_count_host, int64_t n_expert, int n_chunks,
                                       int64_t d_model, int64_t d_hidden, int compute_units, int64_t *bounds_host) {
    FMOE_REQUIRE(expert_count_host && bounds_host && n_expert >= 1, "fmoe_fused_chunk_bounds: bad argument");
    FMOE_REQUIRE(n_chunks >= 0 && n_chunks <= kMaxChunks, "fmoe_fused_chunk_bounds: n_chunks=%d (0..%d)", n_chunks,
                 kMaxChunks);
    FMOE_REQUIRE(d_model >= 1 && d_hidden >= 1 && compute_units >= 0, "fmoe_fused_chunk_bounds: bad sizes");
    int64_t rows = 0;
    for (int64_t e = 0; e < n_expert; ++e) {
        FMOE_REQUIRE(expert_count_host[e] >= 0, "fmoe_fused_chunk_bounds: negative expert count");
        rows += expert_count_host[e];
    }
    const int cus = compute_units > 0 ? compute_units : compute_units_or_default();
    if (n_chunks == 0) {
        // the library's own choice: bounds of that many chunks, the entries up to kAutoChunks repeat the end
        const int n = auto_chunks(expert_count_host, n_expert, d_model, d_hidden, cus);
        chunk_bounds(expert_count_host, n_expert, rows, n, d_model, d_hidden, cus, bounds_host);
        for (int c = n + 1; c <= kAutoChunks; ++c) bounds_host[c] = rows;
        return FMOE_OK;
    }
    chunk_bounds(expert_count_host, n_expert, rows, n_chunks, d_model, d_hidden, cus, bounds_host);
    return FMOE_OK;
}

extern "C" int fmoe_fused_scatter_in_loader(const fmoe_mlp_params *p, const void *inp, int64_t n_tokens) {
    if (p == nullptr || inp == nullptr || n_tokens < 0) return 0;
    // the output pointers only matter for their alignment; torch allocations are 256-byte aligned
    LinearForwardArgs probe{inp, p->w1, p->b1, nullptr, nullptr, p->d_model, p->d_hidden, p->dtype, kEpiBiasAct,
                            p->activation, nullptr, 1, n_tokens};
    return linear_forward_can_gather(probe) ? 1 : 0;
}

extern "C" int fmoe_fused_mlp_forward(const fmoe_mlp_params *p, const void *inp, const int64_t *pos,
                                      const int64_t *slot_to_row, const int64_t *expert_count_host,
                                      int64_t n_tokens, int64_t top_k, int64_t n_rows, void *buf_in,
                                      void *buf_pre, void *buf_mid, void *buf_out, void *out, int n_chunks,
                                      void *stream) {
    if (int rc = check_common("fmoe_fused_mlp_forward", p, expert_count_host, n_tokens, top_k, n_rows, n_chunks))
        return rc;
    const int64_t n_slots = n_tokens * top_k;
    if (n_slots == 0) return FMOE_OK;
    FMOE_REQUIRE(slot_to_row || !out, "fmoe_fused_mlp_forward: NULL slot_to_row");
    FMOE_REQUIRE(n_rows == 0 || (inp && pos && buf_mid && buf_out), "fmoe_fused_mlp_forward: NULL buffer");
    const int dt = p->dtype;
    const int64_t d = p->d_model, h = p->d_hidden, E = p->n_expert;
    hipStream_t caller = (hipStream_t)stream;
    DeviceLanes *l;
    if (int rc = get_lanes(&l)) return rc;
    std::lock_guard<std::mutex> enqueue_lock(g_enqueue_mutex[l - g_lanes]);
    const int cus = compute_units_or_default();
    if (n_chunks == 0) n_chunks = auto_chunks(expert_count_host, E, d, h, cus);
    const CallStreams cs = n_chunks > 1 ? CallStreams{l->in, l->compute, l->out, true} : CallStreams{caller, caller, caller, false};
    if (cs.lanes)
        if (int rc = fork_lanes(l, caller)) return rc;
    int64_t bounds[kMaxChunks + 1];
    chunk_bounds(expert_count_host, E, n_rows, n_chunks, d, h, cus, bounds);

    // dropped slots become zero rows; independent of everything else
    if (out && n_rows < n_slots)
        if (int rc = permute_zero_unmapped(slot_to_row, out, n_slots, d, dt, cs.out)) return rc;

    // The first GEMM reads the token rows through pos in its loader where it can; buf_in is then
    // neither written nor needed (the caller passes NULL).
    LinearForwardArgs probe{inp, p->w1, p->b1, buf_mid, buf_pre, d, h, dt, kEpiBiasAct, p->activation, pos, top_k, n_tokens};
    const bool in_loader = buf_in == nullptr;
    FMOE_REQUIRE(!in_loader || n_rows == 0 || linear_forward_can_gather(probe),
                 "fmoe_fused_mlp_forward: buf_in is NULL but this shape needs the scattered copy "
                 "(ask fmoe_fused_scatter_in_loader first)");
    for (int c = 0; c < n_chunks && !in_loader; ++c) {
        const int64_t lo = bounds[c], hi = bounds[c + 1];
        if (hi == lo) continue;
        // permute-in: buf_in[r] = inp[pos[r] / top_k]
        if (int rc = permute_gather_rows(inp, pos + lo, top_k, at(buf_in, lo, d, dt), hi - lo, n_tokens, d, dt, cs.in))
            return rc;
        if (int rc = record(cs, l->in_ready[c], cs.in)) return rc;
    }
    for (int c = 0; c < n_chunks; ++c) {
        const int64_t lo = bounds[c], hi = bounds[c + 1];
        if (hi == lo) continue;
        if (!in_loader)
            if (int rc = wait(cs, cs.compute, l->in_ready[c])) return rc;
        LinearForwardArgs f1{buf_in, p->w1, p->b1, buf_mid, buf_pre, d, h, dt, kEpiBiasAct, p->activation};
        if (int rc = grouped_linear_forward(in_loader ? probe : f1, expert_count_host, E, lo, hi, cs.compute)) return rc;
        LinearForwardArgs f2{buf_mid, p->w2, p->b2, buf_out, nullptr, h, d, dt, kEpiStore, FMOE_ACT_NONE};
        if (int rc = grouped_linear_forward(f2, expert_count_host, E, lo, hi, cs.compute)) return rc;
        if (int rc = record(cs, l->out_ready[c], cs.compute)) return rc;
    }
    for (int c = 0; c < n_chunks && out; ++c) {
        const int64_t lo = bounds[c], hi = bounds[c + 1];
        if (hi == lo) continue;
        if (int rc = wait(cs, cs.out, l->out_ready[c])) return rc;
        // permute-out: out[pos[r]] = buf_out[r]
        if (int rc = permute_scatter_rows(at(buf_out, lo, d, dt), pos + lo, out, hi - lo, n_slots, d, dt, cs.out))
            return rc;
    }
    return cs.lanes ? join_lanes(l, caller) : FMOE_OK;
}

extern "C" int fmoe_fused_mlp_backward(const fmoe_mlp_params *p, const void *grad_out, const int64_t *pos,
                                       const int64_t *slot_to_row, const int64_t *expert_count_host,
                                       int64_t n_tokens, int64_t top_k, int64_t n_rows, const void *inp,
                                       void *buf_in, const void *buf_pre, const void *buf_mid, void *g_out, void *g_mid,
                                       void *g_in, void *grad_inp, void *grad_w1, void *grad_b1, void *grad_w2,
                                       void *grad_b2, int n_chunks, void *stream) {
    if (int rc = check_common("fmoe_fused_mlp_backward", p, expert_count_host, n_tokens, top_k, n_rows, n_chunks))
        return rc;
    FMOE_REQUIRE(grad_w1 && grad_w2, "fmoe_fused_mlp_backward: NULL weight gradient");
    FMOE_REQUIRE(n_tokens == 0 || (grad_inp && slot_to_row), "fmoe_fused_mlp_backward: NULL grad_inp / slot_to_row");
    FMOE_REQUIRE(n_rows == 0 || ((pos || !grad_out) && buf_in && buf_mid && g_out && g_mid && g_in),
                 "fmoe_fused_mlp_backward: NULL buffer");
    FMOE_REQUIRE(p->activation == FMOE_ACT_NONE || n_rows == 0 || buf_pre,
                 "fmoe_fused_mlp_backward: pre-activation buffer is NULL");
    const int dt = p->dtype;
    const int64_t d = p->d_model, h = p->d_hidden, E = p->n_expert;
    const int64_t n_slots = n_tokens * top_k;
    hipStream_t caller = (hipStream_t)stream;
    DeviceLanes *l;
    if (int rc = get_lanes(&l)) return rc;
    std::lock_guard<std::mutex> enqueue_lock(g_enqueue_mutex[l - g_lanes]);
    const int cus = compute_units_or_default();
    if (n_chunks == 0) n_chunks = auto_chunks(expert_count_host, E, d, h, cus);
    const CallStreams cs = n_chunks > 1 ? CallStreams{l->in, l->compute, l->out, true} : CallStreams{caller, caller, caller, false};
    if (cs.lanes)
        if (int rc = fork_lanes(l, caller)) return rc;
    int64_t bounds[kMaxChunks + 1];
    chunk_bounds(expert_count_host, E, n_rows, n_chunks, d, h, cus, bounds);

    for (int c = 0; c < n_chunks; ++c) {
        const int64_t lo = bounds[c], hi = bounds[c + 1];
        if (hi == lo) continue;
        // permute-in: g_out[r] = grad_out[pos[r]] (nothing to do when the caller filled g_out)
        if (grad_out)
            if (int rc = permute_gather_rows(grad_out, pos + lo, 1, at(g_out, lo, d, dt), hi - lo, n_slots, d, dt, cs.in))
                return rc;
        if (int rc = record(cs, l->in_ready[c], cs.in)) return rc;
    }
    // A forward that read the token rows in its loader kept no sorted copy of the input; the first
    // linear's weight gradient contracts over sorted rows, so the copy is made now (inp != NULL),
    // on the permute-in lane behind the chunks' gradient rows (which the data gradients wait for),
    // long before that product runs.
    if (inp != nullptr && n_rows > 0) {
        FMOE_REQUIRE(pos != nullptr, "fmoe_fused_mlp_backward: pos is NULL");
        if (int rc = permute_gather_rows(inp, pos, top_k, buf_in, n_rows, n_tokens, d, dt, cs.in)) return rc;
    }
    if (int rc = record(cs, l->regather, cs.in)) return rc;
    // Per chunk, only the products a later stage waits for: the two data gradients.
    const bool has_act = p->activation != FMOE_ACT_NONE;
    for (int c = 0; c < n_chunks; ++c) {
        const int64_t lo = bounds[c], hi = bounds[c + 1];
        if (hi == lo) continue;
        if (int rc = wait(cs, cs.compute, l->in_ready[c])) return rc;
        // g_mid = (g_out . W2) * act'(pre);  g_in = g_mid . W1
        LinearDgradArgs d2{g_out, p->w2, g_mid, has_act ? buf_pre : nullptr, h, d, dt,
                           has_act ? kEpiDAct : kEpiStore, p->activation};
        if (int rc = grouped_linear_dgrad(d2, expert_count_host, E, lo, hi, cs.compute)) return rc;
        LinearDgradArgs d1{g_mid, p->w1, g_in, nullptr, d, h, dt, kEpiStore, FMOE_ACT_NONE};
        if (int rc = grouped_linear_dgrad(d1, expert_count_host, E, lo, hi, cs.compute)) return rc;
    }
    // grad_inp[t] = sum of the token's k expert-row gradients (rows of different chunks, so
    // this runs once, after all of them) -- on the permute-out lane, beside the weight gradients
    if (int rc = record(cs, l->out_ready[0], cs.compute)) return rc;
    if (int rc = wait(cs, cs.out, l->out_ready[0])) return rc;
    if (n_tokens > 0)
        if (int rc = fmoe_reduce_slots(g_in, slot_to_row, grad_inp, n_tokens, top_k, n_rows, d, dt, cs.out)) return rc;
    // The weight gradients contract over an expert's rows, all of which exist now: one launch
    // per linear over all rows, so an expert's gradient is accumulated in fp32 from start to end
    // and rounded once, whatever the chunking (experts without rows are zero-filled):
    // gW2 = g_out^T . mid, gb2 = colsum(g_out);  gW1 = g_mid^T . buf_in, gb1 = colsum(g_mid)
    // (the bias gradients come out of the weight-gradient kernel's first column tiles).
    LinearWgradArgs w2{g_out, buf_mid, grad_w2, grad_b2, h, d, dt};
    if (int rc = grouped_linear_wgrad(w2, expert_count_host, E, 0, n_rows, true, cs.compute)) return rc;
    if (int rc = wait(cs, cs.compute, l->regather)) return rc;
    LinearWgradArgs w1{g_mid, buf_in, grad_w1, grad_b1, d, h, dt};
    if (int rc = grouped_linear_wgrad(w1, expert_count_host, E, 0, n_rows, true, cs.compute)) return rc;
    return cs.lanes ? join_lanes(l, caller) : FMOE_OK;
}
