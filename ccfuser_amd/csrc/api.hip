// Whole-layer entry points and error plumbing of libccfuser_moe.so.
//
// ccf_moe_forward strings the stages together on one stream with no host
// synchronisation: gate -> count/scan/pos -> FFN1 -> FFN2 -> combine.  It is
// the one-GPU form of MixMOETransformerMLP.forward
// (mix_moe/mix_moe/transformer.py:475-497) and of _MixMOE::forward
// (mix_moe/csrc/mix_moe.h:507-598).  Where the reference keeps an NVSHMEM
// symmetric heap of 2*tokens*hidden halves as its dispatch buffer
// (mix_moe.h:77), this path needs no dispatch buffer at all (tokens are read
// in place through the row index) and keeps only the activation h and the
// un-permuted expert output in a caller-owned HBM workspace.
#include "ccf_common.h"
#include "plan.h"

namespace ccf {

char *error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

namespace {

// Carves 256-byte aligned pieces out of a caller-owned workspace.
struct Carver {
  char *base;
  size_t used = 0;
  explicit Carver(void *p) : base(static_cast<char *>(p)) {}
  template <typename T>
  T *take(size_t count) {
    T *p = base ? reinterpret_cast<T *>(base + used) : nullptr;
    used += round_up(sizeof(T) * count, 256);
    return p;
  }
};

struct MoeWs {
  int64_t *idx;        // [n_flat] gate output
  int64_t *idx_kept;   // [n_flat]
  half_t *score;       // [n_flat]
  int32_t *counts;     // [E]
  int32_t *offsets;    // [E+1]
  int64_t *pos;        // [n_flat]
  int32_t *src_row, *dst_row, *inv_pos;   // [n_flat] each
  char *route_ws;
  size_t route_bytes;
  char *ffn_ws;
  size_t ffn_bytes;
  half_t *h;           // [n_flat, f]
  half_t *y_flat;      // [n_flat, d]
  size_t total;
};

MoeWs carve_moe(void *ws, int tokens, int d, int f, int E, int k) {
  const size_t n = static_cast<size_t>(tokens) * k;
  Carver c(ws);
  MoeWs w;
  w.idx = c.take<int64_t>(n);
  w.idx_kept = c.take<int64_t>(n);
  w.score = c.take<half_t>(n);
  w.counts = c.take<int32_t>(E);
  w.offsets = c.take<int32_t>(E + 1);
  w.pos = c.take<int64_t>(n);
  w.src_row = c.take<int32_t>(n);
  w.dst_row = c.take<int32_t>(n);
  w.inv_pos = c.take<int32_t>(n);
  w.route_bytes = ccf_route_workspace_bytes(static_cast<int>(n), E);
  w.route_ws = c.take<char>(w.route_bytes);
  w.ffn_bytes = ccf_ffn_workspace_bytes(static_cast<int>(n), E, d, f);
  w.ffn_ws = c.take<char>(w.ffn_bytes);
  w.h = c.take<half_t>(n * f);
  w.y_flat = c.take<half_t>(n * d);
  w.total = c.used;
  return w;
}

struct SegWs {
  int32_t *counts, *offsets, *rows;
  char *ffn_ws;
  size_t ffn_bytes;
  half_t *h;
  size_t total;
};

SegWs carve_seg(void *ws, int total_rows, int d, int f, int E) {
  Carver c(ws);
  SegWs w;
  w.counts = c.take<int32_t>(E);
  w.offsets = c.take<int32_t>(E + 1);
  w.rows = c.take<int32_t>(total_rows);
  w.ffn_bytes = ccf_ffn_workspace_bytes(total_rows, E, d, f);
  w.ffn_ws = c.take<char>(w.ffn_bytes);
  w.h = c.take<half_t>(static_cast<size_t>(total_rows) * f);
  w.total = c.used;
  return w;
}

// Optional per-stage timing: events recorded on the layer's stream before the
// gate and after each of the five stages of the next ccf_moe_forward calls
// (ccf_moe_ffn_segments records the same six; its gate and combine stages are empty).
thread_local hipEvent_t g_stage_events[6];
thread_local int g_stage_event_count = 0;

inline void mark_stage(int i, hipStream_t st) {
  if (i < g_stage_event_count && g_stage_events[i]) (void)hipEventRecord(g_stage_events[i], st);
}

bool sizes_ok(long long rows, int d, int f) {
  // row offsets are formed in 64 bits, but the row tables are int32
  return rows >= 0 && rows < (1ll << 31) && d > 0 && f > 0;
}

}  // namespace
}  // namespace ccf

extern "C" int ccf_version(void) { return 100; }

extern "C" const char *ccf_last_error(void) { return ccf::error_buffer(); }

extern "C" int ccf_moe_forward_set_events(void *const *events, int count) {
  using namespace ccf;
  CCF_REQUIRE(count >= 0 && count <= 6 && (events || count == 0), CCF_ERR_ARG,
              "moe_forward_set_events: count %d outside 0..6", count);
  for (int i = 0; i < count; ++i) g_stage_events[i] = static_cast<hipEvent_t>(events[i]);
  g_stage_event_count = count;
  return CCF_OK;
}

extern "C" size_t ccf_moe_workspace_bytes(int tokens, int d_model, int d_ffn, int num_expert,
                                          int top_k) {
  if (tokens < 0 || d_model <= 0 || d_ffn <= 0 || num_expert <= 0 || top_k <= 0) return 0;
  if (static_cast<long long>(tokens) * top_k >= (1ll << 31)) return 0;
  return ccf::carve_moe(nullptr, tokens, d_model, d_ffn, num_expert, top_k).total;
}

extern "C" int ccf_moe_forward(const void *x, const void *wg, const void *bg, const void *w1,
                               const void *b1, const void *w2, const void *b2, int tokens,
                               int d_model, int d_ffn, int num_expert, int top_k, int capacity,
                               void *out, int64_t *idx_out, void *score_out, int64_t *pos_out,
                               int32_t *counts_out, int32_t *offsets_out, void *workspace,
                               size_t workspace_bytes, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(x && wg && w1 && b1 && w2 && b2 && out, CCF_ERR_ARG, "moe_forward: null pointer");
  CCF_REQUIRE(tokens >= 0 && num_expert > 0 && top_k >= 1, CCF_ERR_ARG, "moe_forward: bad size");
  CCF_REQUIRE(sizes_ok(static_cast<long long>(tokens) * top_k, d_model, d_ffn), CCF_ERR_SHAPE,
              "moe_forward: tokens*top_k too large");
  const size_t need = ccf_moe_workspace_bytes(tokens, d_model, d_ffn, num_expert, top_k);
  CCF_REQUIRE(workspace && workspace_bytes >= need, CCF_ERR_WORKSPACE,
              "moe_forward: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  if (tokens == 0) return CCF_OK;
  MoeWs w = carve_moe(workspace, tokens, d_model, d_ffn, num_expert, top_k);
  // counts and offsets are written straight into the caller's arrays when given
  if (counts_out) w.counts = counts_out;
  if (offsets_out) w.offsets = offsets_out;
  const int n = tokens * top_k;
  hipStream_t st = as_stream(stream);
  int rc;
  mark_stage(0, st);
  // the gate's selection threads also leave per-workgroup expert counts in the routing workspace when that
  // table is small and a workgroup's flat indices tile the routing chunks (top_k a power of two): the
  // routing stage is then one launch
  int gate_tokens = 0;
  const bool pow2_k = (top_k & (top_k - 1)) == 0;
  if ((rc = gate_forward(x, wg, bg, tokens, d_model, num_expert, top_k, CCF_F16, w.idx, w.score, nullptr, stream,
                         pow2_k ? reinterpret_cast<int32_t *>(w.route_ws) : nullptr, route_rows_max_ints(), &gate_tokens)))
    return rc;
  mark_stage(1, st);
  // the tile plans of both GEMMs are built by two more workgroups of the routing stage's last
  // launch (they need the offsets only), which saves the GEMMs a small launch each
  PlanReq plans[2];
  const GemmOptions opt = forward_options();        // one snapshot for the plans and the GEMMs that consume them
  // top-1 without a capacity limit: every token has one slot, its score is exactly 1 (the softmax of
  // one logit) and its flat row is its token row, so FFN2 writes the layer output itself
  const bool direct = top_k == 1 && capacity < 0;
  // top-2 with the option on: FFN2's epilogue adds score * y into the zero-filled output
  const bool fuse = opt.fused_combine && top_k == 2 && d_model % 8 == 0;
  const bool planned = forward_plan_request(1, n, num_expert, d_model, d_ffn, w.ffn_ws, opt, &plans[0]) &&
                       forward_plan_request(fuse ? 3 : 2, n, num_expert, d_model, d_ffn, w.ffn_ws, opt, &plans[1]);
  if ((rc = route_with_plans(w.idx, n, num_expert, top_k, capacity, w.counts, w.offsets, w.pos, w.src_row,
                             w.dst_row, w.inv_pos, w.idx_kept, w.route_ws, w.route_bytes, st, plans,
                             planned ? 2 : 0, gate_tokens * top_k)))
    return rc;
  mark_stage(2, st);
  if ((rc = ffn1_forward(x, w.src_row, nullptr, w.offsets, n, num_expert, d_model, d_ffn, w1, b1, 1, w.h,
                         w.ffn_ws, w.ffn_bytes, st, planned ? &opt : nullptr)))
    return rc;
  mark_stage(3, st);
  if (fuse) {
    if ((rc = launch_zero(static_cast<half_t *>(out), static_cast<size_t>(tokens) * d_model, st))) return rc;
    if ((rc = ffn2_forward_combine(w.h, w.src_row, w.dst_row, w.offsets, n, num_expert, d_model, d_ffn, w2, b2,
                                   w.score, out, w.ffn_ws, w.ffn_bytes, st, planned ? &opt : nullptr)))
      return rc;
    mark_stage(4, st);
  } else if ((rc = ffn2_forward(w.h, nullptr, w.dst_row, w.offsets, n, num_expert, d_model, d_ffn, w2, b2,
                         nullptr, direct ? out : w.y_flat, w.ffn_ws, w.ffn_bytes, st, planned ? &opt : nullptr)))
    return rc;
  if (!fuse) mark_stage(4, st);
  if (!direct && !fuse) {
    if ((rc = ccf_combine(w.y_flat, w.score, w.inv_pos, out, tokens, top_k, d_model, stream)))
      return rc;
  }
  mark_stage(5, st);
  // optional copies of the routing results (device to device, same stream)
  hipError_t e = hipSuccess;
  if (idx_out && e == hipSuccess)
    e = hipMemcpyAsync(idx_out, w.idx_kept, sizeof(int64_t) * n, hipMemcpyDeviceToDevice, st);
  if (score_out && e == hipSuccess)
    e = hipMemcpyAsync(score_out, w.score, sizeof(half_t) * n, hipMemcpyDeviceToDevice, st);
  if (pos_out && e == hipSuccess)
    e = hipMemcpyAsync(pos_out, w.pos, sizeof(int64_t) * n, hipMemcpyDeviceToDevice, st);
  if (e != hipSuccess) return fail(CCF_ERR_HIP, "moe_forward: copy failed: %s", hipGetErrorString(e));
  return CCF_OK;
}

extern "C" size_t ccf_segments_workspace_bytes(int total_rows, int n_seg, int num_expert,
                                               int d_model, int d_ffn) {
  if (total_rows < 0 || n_seg < 0 || num_expert <= 0 || d_model <= 0 || d_ffn <= 0) return 0;
  return ccf::carve_seg(nullptr, total_rows, d_model, d_ffn, num_expert).total;
}

extern "C" int ccf_moe_ffn_segments(const void *x, const int32_t *seg_start, const int32_t *seg_len,
                                    const int32_t *seg_expert, int n_seg, int total_rows,
                                    int d_model, int d_ffn, int num_expert, const void *w1,
                                    const void *b1, const void *w2, const void *b2, void *y,
                                    void *workspace, size_t workspace_bytes, ccf_stream_t stream) {
  using namespace ccf;
  CCF_REQUIRE(x && seg_start && seg_len && seg_expert && w1 && b1 && w2 && b2 && y, CCF_ERR_ARG,
              "moe_ffn_segments: null pointer");
  CCF_REQUIRE(n_seg >= 0 && total_rows >= 0 && num_expert > 0, CCF_ERR_ARG,
              "moe_ffn_segments: bad size");
  const size_t need = ccf_segments_workspace_bytes(total_rows, n_seg, num_expert, d_model, d_ffn);
  CCF_REQUIRE(workspace && workspace_bytes >= need, CCF_ERR_WORKSPACE,
              "moe_ffn_segments: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  if (total_rows == 0 || n_seg == 0) return CCF_OK;
  SegWs w = carve_seg(workspace, total_rows, d_model, d_ffn, num_expert);
  hipStream_t st = as_stream(stream);
  int rc;
  mark_stage(0, st);
  mark_stage(1, st);                                  // no gate in this call
  // the tile plans of both GEMMs are built by more workgroups of the regrouping launch, as in ccf_moe_forward
  PlanReq plans[2];
  const GemmOptions opt = forward_options();
  const bool planned = forward_plan_request(1, total_rows, num_expert, d_model, d_ffn, w.ffn_ws, opt, &plans[0]) &&
                       forward_plan_request(2, total_rows, num_expert, d_model, d_ffn, w.ffn_ws, opt, &plans[1]);
  if ((rc = segments_with_plans(seg_start, seg_len, seg_expert, n_seg, num_expert, total_rows, w.counts, w.offsets,
                                w.rows, st, plans, planned ? 2 : 0)))
    return rc;
  mark_stage(2, st);
  if ((rc = ffn1_forward(x, w.rows, nullptr, w.offsets, total_rows, num_expert, d_model, d_ffn, w1, b1, 1,
                         w.h, w.ffn_ws, w.ffn_bytes, st, planned ? &opt : nullptr)))
    return rc;
  mark_stage(3, st);
  rc = ffn2_forward(w.h, nullptr, w.rows, w.offsets, total_rows, num_expert, d_model, d_ffn, w2, b2,
                    nullptr, y, w.ffn_ws, w.ffn_bytes, st, planned ? &opt : nullptr);
  mark_stage(4, st);
  mark_stage(5, st);                                  // no combine either
  return rc;
}
