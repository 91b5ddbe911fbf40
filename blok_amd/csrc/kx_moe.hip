// kx_moe.hip -- one routed-MoE decode layer for T tokens.
//
// Reference: the MoE branch of run(), src/kimi_exec.cu:835-877 -- router gate
// matvec (fp32 logits), sigmoid + bias + top-8, a blocking copy of the 8 ids to
// the host, then per slot 32+112 tile launches each preceded by NVMe reads,
// expert_accum_k per tile, round_bf16_k, the shared expert through bf16_mlp and
// the residual add.  Here, no host round trip, and for up to 4 tokens four launches:
//   1 shared gate+up bf16 GEMV with SwiGLU (-> smid [T, shared_inter]) and the router's logits
//     GEMV in one launch; the router workgroup that finishes last does sigmoid/bias/top-k and
//     the bucketing (pairs sorted by expert, list of active experts)
//   2 routed gate+up INT4 GEMV with the SwiGLU epilogue   -> mid  [T*topk, moe_inter]
//   3 routed down INT4 GEMV                               -> eout [T*topk, hidden]
//   4 shared down bf16 GEMV; epilogue combines the topk routed outputs in slot
//     order, adds the shared output and the residual.
// For one token 3 and 4 are one launch: every workgroup of the routed down GEMV goes on to a chunk
// of the shared down GEMV, and the workgroup that completes a block of output rows combines it.
// More tokens: router GEMV, top-k + bucketing, and the shared gate+up GEMV are launches of
// their own; beyond T*topk = E pairs the routed kernels run as two launches each (experts
// with one pair, experts with more).
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_front.h"

constexpr int KX_TAIL_BLOCKS = 1024;

struct kx_moe_workspace {
  int max_tokens;
  kx_config cfg;
  float *logits;      // [T, E]
  uint16_t *ids;      // [T, topk]
  float *weights;     // [T, topk]
  int *counts;        // [E]
  int *offsets;       // [E+1]
  int *pairs;         // [T*topk]
  int4 *work;         // [E] {expert, first, last, first pair}
  int4 *pair_work;    // [T*topk] one record per pair {expert, q, q + 1, pairs[q]}
  int *n_active;      // [1]
  int *route_counter; // [10] zero between launches: workgroups of the router GEMV count themselves in (one counter, or one and one per block of four tokens)
  int *tail_count;    // [KX_TAIL_BLOCKS] zero between launches: arrivals per block of output rows (routed down + shared down)
  uint16_t *mid;      // [T*topk, moe_inter]
  uint16_t *eout;     // [T*topk, hidden]
  uint16_t *smid;     // [T, shared_inter]
  uint16_t *sy;       // [T, hidden] shared expert output (prefill path)
  uint32_t *mid_hand; // [topk, moe_inter] tagged words: one token's mid values inside the resident routed launch
  uint32_t mid_tag = 0;
  int *err = nullptr; // the caller's flag for waits given up inside resident launches (not owned)
  hipEvent_t ev[6];
  // a second stream for the batched forms: the experts with one pair (GEMV kernels) and the shared expert run beside the
  // grouped GEMMs of the experts with several pairs instead of in front of them.  Default priority, like every stream here.
  hipStream_t side = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
};

static int check_cfg(const kx_config *c) {
  KX_REQUIRE(c, "kx_moe: null config");
  KX_REQUIRE(c->hidden > 0 && c->hidden % 1024 == 0, "kx_moe: hidden=%d must be a multiple of 1024", c->hidden);
  KX_REQUIRE(c->moe_inter > 0 && c->moe_inter % 1024 == 0, "kx_moe: moe_inter=%d must be a multiple of 1024", c->moe_inter);
  KX_REQUIRE(c->shared_inter > 0 && c->shared_inter % 512 == 0, "kx_moe: shared_inter=%d must be a multiple of 512", c->shared_inter);
  KX_REQUIRE(c->experts > 0 && c->experts <= 1024, "kx_moe: experts=%d outside [1, 1024]", c->experts);
  KX_REQUIRE(c->topk > 0 && c->topk <= c->experts && c->topk <= 64, "kx_moe: topk=%d outside [1, min(64, experts)]", c->topk);
  return KX_OK;
}

extern "C" int kx_moe_workspace_create(const kx_config *cfg, int32_t max_tokens, kx_moe_workspace **out) {
  KX_REQUIRE(out, "kx_moe_workspace_create: null out pointer");
  *out = nullptr;
  int rc = check_cfg(cfg);
  if (rc) return rc;
  KX_REQUIRE(max_tokens > 0, "kx_moe_workspace_create: max_tokens=%d must be positive", max_tokens);
  kx_moe_workspace *ws = new kx_moe_workspace();
  ws->max_tokens = max_tokens;
  ws->cfg = *cfg;
  const size_t T = (size_t)max_tokens, E = (size_t)cfg->experts, K = (size_t)cfg->topk;
  struct { void **p; size_t bytes; } allocs[] = {
      {(void **)&ws->logits, T * E * 4}, {(void **)&ws->ids, T * K * 2}, {(void **)&ws->weights, T * K * 4},
      {(void **)&ws->counts, E * 4}, {(void **)&ws->offsets, (E + 1) * 4}, {(void **)&ws->pairs, T * K * 4},
      {(void **)&ws->work, E * 16}, {(void **)&ws->pair_work, T * K * 16}, {(void **)&ws->n_active, 64}, {(void **)&ws->tail_count, KX_TAIL_BLOCKS * 4},
      {(void **)&ws->mid, T * K * (size_t)cfg->moe_inter * 2}, {(void **)&ws->eout, T * K * (size_t)cfg->hidden * 2},
      {(void **)&ws->smid, T * (size_t)cfg->shared_inter * 2}, {(void **)&ws->sy, T * (size_t)cfg->hidden * 2},
      {(void **)&ws->mid_hand, K * (size_t)cfg->moe_inter * 4}};
  for (auto &al : allocs) {
    hipError_t e = hipMalloc(al.p, al.bytes);
    if (e != hipSuccess) {
      kx_set_error("kx_moe_workspace_create: hipMalloc(%zu): %s", al.bytes, hipGetErrorString(e));
      kx_moe_workspace_destroy(ws);
      return KX_ERR_HIP;
    }
  }
  ws->route_counter = ws->n_active + 1;
  // work records nobody has written yet say "no expert" (-1): kx_moe_routed_only before any layer call, or with more
  // tokens than the last one had, then does nothing instead of following uninitialised records
  hipError_t e = hipMemset(ws->work, 0xff, E * 16);
  if (e == hipSuccess) e = hipMemset(ws->pair_work, 0xff, T * K * 16);
  if (e == hipSuccess) e = hipMemset(ws->n_active, 0, 64);
  if (e == hipSuccess) e = hipMemset(ws->tail_count, 0, KX_TAIL_BLOCKS * 4);
  if (e == hipSuccess) e = hipMemset(ws->mid_hand, 0, K * (size_t)cfg->moe_inter * 4);
  for (auto &ev : ws->ev)
    if (e == hipSuccess) e = hipEventCreate(&ev);
  if (e == hipSuccess) e = hipStreamCreateWithFlags(&ws->side, hipStreamNonBlocking);
  if (e == hipSuccess) e = hipEventCreateWithFlags(&ws->fork, hipEventDisableTiming);
  if (e == hipSuccess) e = hipEventCreateWithFlags(&ws->join, hipEventDisableTiming);
  if (e != hipSuccess) {
    kx_set_error("kx_moe_workspace_create: %s", hipGetErrorString(e));
    kx_moe_workspace_destroy(ws);
    return KX_ERR_HIP;
  }
  *out = ws;
  return KX_OK;
}

extern "C" int kx_moe_workspace_destroy(kx_moe_workspace *ws) {
  if (!ws) return KX_OK;
  void *ptrs[] = {ws->logits, ws->ids, ws->weights, ws->counts, ws->offsets, ws->pairs,
                  ws->work, ws->pair_work, ws->n_active, ws->tail_count, ws->mid, ws->eout, ws->smid, ws->sy, ws->mid_hand};
  for (void *p : ptrs)
    if (p) (void)hipFree(p);
  for (auto &e : ws->ev)
    if (e) (void)hipEventDestroy(e);
  if (ws->side) { (void)hipStreamSynchronize(ws->side); (void)hipStreamDestroy(ws->side); }
  if (ws->fork) (void)hipEventDestroy(ws->fork);
  if (ws->join) (void)hipEventDestroy(ws->join);
  delete ws;
  return KX_OK;
}

int *kx_moe_workspace_n_active(kx_moe_workspace *ws) { return ws->n_active; }
void kx_moe_workspace_set_err(kx_moe_workspace *ws, int *d_err) { ws->err = d_err; }

void kx_moe_head_args(const kx_config *c, const kx_moe_weights *w, kx_moe_workspace *ws, void *d_n, const uint16_t *norm_w, KxMoeHeadArgs *out) {
  KxMoeHeadArgs h = {};
  h.post_ln = norm_w;
  h.w_gate = (const uint16_t *)w->d_shared_gate; h.w_up = (const uint16_t *)w->d_shared_up; h.w_router = (const uint16_t *)w->d_router_gate;
  h.bias = (const float *)w->d_router_bias;
  h.n_out = (uint16_t *)d_n; h.smid = ws->smid; h.logits = ws->logits; h.ids = ws->ids; h.weights = ws->weights;
  h.counts = ws->counts; h.offsets = ws->offsets; h.pairs = ws->pairs; h.work = ws->work; h.n_active = ws->n_active;
  h.shared_inter = c->shared_inter; h.experts = c->experts; h.topk = c->topk; h.routed_scale = c->routed_scale; h.eps = c->rms_eps;
  *out = h;
}

extern "C" int kx_moe_workspace_views(kx_moe_workspace *ws, void **d_logits, void **d_ids, void **d_weights,
                                      void **d_counts, void **d_offsets, void **d_pairs, void **d_mid,
                                      void **d_expert_out) {
  KX_REQUIRE(ws, "kx_moe_workspace_views: null workspace");
  if (d_logits) *d_logits = ws->logits;
  if (d_ids) *d_ids = ws->ids;
  if (d_weights) *d_weights = ws->weights;
  if (d_counts) *d_counts = ws->counts;
  if (d_offsets) *d_offsets = ws->offsets;
  if (d_pairs) *d_pairs = ws->pairs;
  if (d_mid) *d_mid = ws->mid;
  if (d_expert_out) *d_expert_out = ws->eout;
  return KX_OK;
}

// How the routed kernels go over the experts.  Every pass over an expert streams its weights again, so an expert
// with n pairs wants n tokens per pass; more tokens per pass cost registers and speed.  Up to T*topk = E pairs one
// launch with one token per pass is fastest (measured: splitting pays from about 48 tokens on); beyond that the
// experts with one pair take the one-token kernel and the others a second launch with 2 (or 4) tokens per pass.
struct RoutedPlan {
  int n, tt[2], lo[2], hi[2];
};
static RoutedPlan routed_plan(int tokens, int topk, int experts) {
  const long pairs = (long)tokens * topk;
  RoutedPlan p;
  if (pairs <= experts) {
    p.n = 1; p.tt[0] = 1; p.lo[0] = 0; p.hi[0] = 0x7fffffff;
  } else {
    p.n = 2;
    p.tt[0] = 1; p.lo[0] = 1; p.hi[0] = 1;
    p.tt[1] = pairs <= 4L * experts ? 2 : 4; p.lo[1] = 2; p.hi[1] = 0x7fffffff;
  }
  return p;
}

// From 2 tokens on (the launch that finishes the layer for one token wants the per-expert list) and while one launch
// with one token per pass is the plan, the routed kernels go over the per-pair work list: one workgroup per (chunk, pair).
// A chunk's workgroups run at the same time on the same L2 (their ids differ by multiples of the chunks per expert,
// a multiple of 8 at Kimi shapes), where one workgroup doing the expert's pairs one after the other streams the chunk
// from memory once per pair (the chunks in flight, 29 MB, do not stay in L2) and is the launch's tail when an expert
// has many pairs.  Batch 32 in the stack: gate/up 670 -> 544 us, down 385 -> 330 us per layer.
static bool routed_per_pair(int tokens, int topk, int experts) { return tokens >= 2 && (long)tokens * topk <= experts; }

// the routed gate/up (which = 0) or down (which = 1) kernel(s) over the work list in the workspace
static int routed_launch(const kx_config *c, const kx_moe_weights *w, kx_moe_workspace *ws, const uint16_t *n, int tokens,
                         int which, hipStream_t st) {
  const int H = c->hidden, I = c->moe_inter, E = c->experts, K = c->topk;
  const int max_active = (long)tokens * K < E ? tokens * K : E;
  const RoutedPlan p = routed_plan(tokens, K, E);
  if (routed_per_pair(tokens, K, E)) {  // one workgroup per (chunk, pair)
    if (which == 0) {
      return kx_i4_launch(true, (const uint32_t *)w->d_gate_packed, (const uint16_t *)w->d_gate_scale,
                          (const uint32_t *)w->d_up_packed, (const uint16_t *)w->d_up_scale, n, ws->mid, ws->pair_work, ws->pairs, 0, I,
                          H, K, (size_t)I * (H / 8), (size_t)I * (H / 32), 1, tokens * K, 0, 0x7fffffff, st,
                          tokens * K >= 128 ? 2 : 1);  // 64-row chunks from 128 pairs on (3 % at 256 pairs, none at 64)
    }
    return kx_i4_launch(false, (const uint32_t *)w->d_down_packed, (const uint16_t *)w->d_down_scale, nullptr, nullptr,
                        ws->mid, ws->eout, ws->pair_work, ws->pairs, 0, H, I, 1, (size_t)H * (I / 8), (size_t)H * (I / 32),
                        1, tokens * K, 0, 0x7fffffff, st, tokens * K >= 32 ? 2 : 1);
  }
  for (int i = 0; i < p.n; ++i) {
    int rc;
    if (which == 0)
      rc = kx_i4_launch(true, (const uint32_t *)w->d_gate_packed, (const uint16_t *)w->d_gate_scale,
                        (const uint32_t *)w->d_up_packed, (const uint16_t *)w->d_up_scale, n, ws->mid, ws->work, ws->pairs, 0, I,
                        H, K, (size_t)I * (H / 8), (size_t)I * (H / 32), p.tt[i], max_active, p.lo[i], p.hi[i], st);
    else
      rc = kx_i4_launch(false, (const uint32_t *)w->d_down_packed, (const uint16_t *)w->d_down_scale, nullptr, nullptr,
                        ws->mid, ws->eout, ws->work, ws->pairs, 0, H, I, 1, (size_t)H * (I / 8), (size_t)H * (I / 32),
                        p.tt[i], max_active, p.lo[i], p.hi[i], st, tokens * K >= 32 ? 2 : 1);
    if (rc) return rc;
  }
  return KX_OK;
}

static int moe_layer_body(const kx_config *c, const kx_moe_weights *w, kx_moe_workspace *ws, void *d_n, void *d_x,
                          int tokens, uint32_t flags, const uint16_t *norm_w, hipStream_t st, bool timed, bool &forked);

// An error after the layer has put work on its side stream must not leave that work unjoined: the caller's stream
// waits for it here, so whatever the caller does next (free the buffers, run the layer again) comes after it.
int kx_moe_layer_launch(const kx_config *c, const kx_moe_weights *w, kx_moe_workspace *ws, void *d_n, void *d_x,
                        int tokens, uint32_t flags, const uint16_t *norm_w, hipStream_t st, bool timed) {
  bool forked = false;
  const int rc = moe_layer_body(c, w, ws, d_n, d_x, tokens, flags, norm_w, st, timed, forked);
  if (rc && forked && hipEventRecord(ws->join, ws->side) == hipSuccess) (void)hipStreamWaitEvent(st, ws->join, 0);
  return rc;
}

static int moe_layer_body(const kx_config *c, const kx_moe_weights *w, kx_moe_workspace *ws, void *d_n, void *d_x,
                          int tokens, uint32_t flags, const uint16_t *norm_w, hipStream_t st, bool timed, bool &forked) {
  int rc = check_cfg(c);
  if (rc) return rc;
  KX_REQUIRE(w && ws && d_n && d_x, "kx_moe_decode_layer: null argument");
  KX_REQUIRE(tokens > 0 && tokens <= ws->max_tokens, "kx_moe_decode_layer: tokens=%d outside [1, %d]", tokens, ws->max_tokens);
  KX_REQUIRE(c->hidden == ws->cfg.hidden && c->moe_inter == ws->cfg.moe_inter && c->experts == ws->cfg.experts &&
                 c->topk == ws->cfg.topk && c->shared_inter == ws->cfg.shared_inter,
             "kx_moe_decode_layer: workspace was created for another shape");
  const int H = c->hidden, E = c->experts, K = c->topk;
  const uint16_t *n = (const uint16_t *)d_n;
  if (timed) KX_HIP(hipEventRecord(ws->ev[0], st));
  // router logits, top-k, bucketing; shared gate/up + SwiGLU.  Up to 4 tokens: one launch for all of it.
  KxGemvArgs g = {};
  g.w0 = (const uint16_t *)w->d_router_gate; g.x = n; g.x_stride = H; g.out = ws->logits; g.out_stride = E;
  g.rows = E; g.cols = H; g.tokens = tokens;
  KxGemvArgs s = {};
  s.w0 = (const uint16_t *)w->d_shared_gate; s.w1 = (const uint16_t *)w->d_shared_up; s.x = n; s.x_stride = H;
  s.out = ws->smid; s.out_stride = c->shared_inter; s.rows = c->shared_inter; s.cols = H; s.tokens = tokens;
  if (norm_w) {  // both GEMVs norm the residual stream themselves; the router leaves the normed rows in d_n
    g.x = (const uint16_t *)d_x; g.norm_w = norm_w; g.norm_eps = c->rms_eps; g.norm_out = (uint16_t *)d_n;
    s.x = (const uint16_t *)d_x; s.norm_w = norm_w; s.norm_eps = c->rms_eps;
  }
  // From 5 tokens on a caller may ask for the shared expert on the matrix cores (another summation order, held to
  // the 1e-2 bar; the router and the routed experts stay as they are, so the routing does not change).  Its two
  // products need nothing from the router or the routed experts: they run on the side stream while this one routes
  // and runs the routed experts, and are joined before the combine.
  const bool mm = (flags & KX_MOE_SHARED_MATRIX_CORES) && tokens >= 5 && tokens <= 32;
  const bool rmm = (flags & KX_MOE_ROUTED_MATRIX_CORES) && tokens >= 5;
  // The grouped GEMMs take the experts with at least three pairs, the GEMV kernels those with one or two: a GEMM
  // workgroup holds a CU for the whole of its 112 K steps whatever its tokens, and at 32 sequences the experts with
  // two pairs made the GEMMs a round of 256 workgroups and a twelfth (measured, batch 32: 1897 tok/s with the line
  // at two pairs, 1983 at three, 1941 at four, 1812 at six; batch 16: 1313 -> 1325; batch 12: level)
  // From 32 to 64 tokens the matrix-core class is run by the kernel that dequantizes in registers (kx_i4mm.hip),
  // which costs about as much as a GEMV pass over the expert whatever its tokens: it takes the experts from two
  // pairs on (batch 32: 2514 tok/s against 2497 with the grouped GEMMs from three pairs and 2435 / 2296 with this
  // kernel from three / one; 64 tokens of the one-layer bench: 1.87 ms against 2.00 ms on the GEMV kernels alone and
  // 2.10 ms with the grouped GEMMs; batch 16: 1526 against 1570, so smaller batches keep the grouped GEMMs).
  const bool i4mm = rmm && tokens >= 32 && tokens <= 64;
  const int rmm_min = i4mm ? 2 : 3;
  bool shared_up_done = false, shared_down_done = false;
  if (mm && !norm_w) {
    KX_HIP(hipEventRecord(ws->fork, st));
    KX_HIP(hipStreamWaitEvent(ws->side, ws->fork, 0));
    forked = true;
    if ((rc = kx_skinny_gemm_launch(true, s.w0, s.w1, s.x, s.x_stride, s.out, s.out_stride, KX_GG_BF16, tokens, s.rows, s.cols,
                                    &shared_up_done, ws->side))) return rc;
    if (shared_up_done &&
        (rc = kx_skinny_gemm_launch(false, (const uint16_t *)w->d_shared_down, nullptr, ws->smid, c->shared_inter, ws->sy, H, KX_GG_BF16,
                                    tokens, H, c->shared_inter, &shared_down_done, ws->side))) return rc;
  }
  bool paired = (flags & KX_MOE_HEAD_DONE) && tokens == 1 && norm_w && !mm;  // the caller's launch has done this step
  if (!paired && (rc = kx_gemv_pair_route_launch(s, g, (const float *)w->d_router_bias, ws->ids, ws->weights, E, K, c->routed_scale,
                                      ws->counts, ws->offsets, ws->pairs, ws->work, ws->n_active, ws->route_counter, &paired,
                                      st, routed_per_pair(tokens, K, E) ? ws->pair_work : nullptr))) return rc;
  if (!paired) {
    bool routed = false;
    if ((rc = kx_gemv_route_launch(g, (const float *)w->d_router_bias, ws->ids, ws->weights, E, K, c->routed_scale, ws->counts,
                                   ws->offsets, ws->pairs, ws->work, ws->n_active, ws->route_counter, &routed, st,
                                   routed_per_pair(tokens, K, E) ? ws->pair_work : nullptr))) return rc;
    if (!routed && (rc = kx_route_launch(ws->logits, (const float *)w->d_router_bias, ws->ids, ws->weights, tokens, E, K, c->routed_scale,
                              ws->counts, ws->offsets, ws->pairs, ws->work, ws->n_active, st,
                              routed_per_pair(tokens, K, E) ? ws->pair_work : nullptr))) return rc;
  }
  if (timed) KX_HIP(hipEventRecord(ws->ev[1], st));
  const int n_slots = (long)tokens * K < E ? tokens * K : E;
  // one token: the routed experts and the layer's tail as one resident launch
  bool resident = false;
  if ((flags & KX_MOE_ROUTED_RESIDENT) && ws->err && paired && tokens == 1 && !(flags & KX_MOE_SEPARATE_TAIL) && H / 16 <= KX_TAIL_BLOCKS) {
    KxGemvArgs d = {};
    d.w0 = (const uint16_t *)w->d_shared_down; d.x = ws->smid; d.x_stride = c->shared_inter; d.out = d_x;
    d.out_stride = H; d.rows = H; d.cols = c->shared_inter; d.tokens = tokens; d.expert_out = ws->eout;
    d.route_w = ws->weights; d.topk = K; d.flags = flags & 1u;
    KxMoeTail t = {};
    t.counter = ws->tail_count; t.n_active = ws->n_active; t.sy = ws->sy; t.route_w = ws->weights; t.x = (uint16_t *)d_x;
    t.x_stride = H; t.tokens = tokens; t.topk = K; t.flags = flags & 1u;
    const uint32_t tag = ws->mid_tag % 65535u + 1u;
    if ((rc = kx_i4_routed_shared_launch((const uint32_t *)w->d_gate_packed, (const uint16_t *)w->d_gate_scale, (const uint32_t *)w->d_up_packed,
                                         (const uint16_t *)w->d_up_scale, (const uint32_t *)w->d_down_packed, (const uint16_t *)w->d_down_scale,
                                         n, ws->mid, ws->eout, ws->work, ws->pairs, H, c->moe_inter, K, n_slots, d, t, ws->mid_hand, tag, ws->err,
                                         &resident, st))) return rc;
    if (resident) {
      ws->mid_tag = tag;
      if (timed)
        for (int i = 2; i <= 5; ++i) KX_HIP(hipEventRecord(ws->ev[i], st));
      return KX_OK;
    }
  }
  // routed gate/up + SwiGLU
  if (rmm) {
    // Experts with one pair: the GEMV kernels (they stream such an expert at their rate); the others: the grouped
    // GEMMs.  The two classes touch different experts and different rows of mid and of the expert outputs, so they
    // run side by side: the GEMV class (gate/up, then down) and after it the shared expert on the side stream, the
    // GEMM class (gate/up, then down) on this one, joined before the combine.  A GEMM workgroup holds a whole CU
    // for its 112 K steps and a batch of 32 brings about 280 of them for 256 CUs; side by side, the other class
    // fills the CUs that the second round of those would leave idle (batch 32: two launches in sequence took
    // 148 + 251 us for gate/up and 77 + 117 us for down).
    const int I = c->moe_inter;
    KX_HIP(hipEventRecord(ws->fork, st));  // the routing is in
    KX_HIP(hipStreamWaitEvent(ws->side, ws->fork, 0));
    forked = true;
    bool mm_done = false;
    if (i4mm &&
        (rc = kx_i4mm_launch(true, (const uint32_t *)w->d_gate_packed, (const uint16_t *)w->d_gate_scale, (const uint32_t *)w->d_up_packed,
                             (const uint16_t *)w->d_up_scale, n, ws->mid, ws->work, ws->pairs, n_slots, I, H, K, (size_t)I * (H / 8),
                             (size_t)I * (H / 32), rmm_min, 1 << 30, kx_cdiv(tokens, 32), &mm_done, st))) return rc;
    if (!mm_done &&
        (rc = kx_grouped_gemm_launch(true, true, w->d_gate_packed, (const uint16_t *)w->d_gate_scale, w->d_up_packed,
                                     (const uint16_t *)w->d_up_scale, n, ws->mid, KX_GG_BF16, ws->work, ws->pairs, 0, n_slots, I, H,
                                     K, (size_t)I * (H / 8), (size_t)I * (H / 32), tokens, st, rmm_min))) return rc;
    if ((rc = kx_i4_launch(true, (const uint32_t *)w->d_gate_packed, (const uint16_t *)w->d_gate_scale,
                           (const uint32_t *)w->d_up_packed, (const uint16_t *)w->d_up_scale, n, ws->mid, ws->work, ws->pairs, 0, I,
                           H, K, (size_t)I * (H / 8), (size_t)I * (H / 32), 1, n_slots, 1, rmm_min - 1, ws->side))) return rc;
  } else if ((rc = routed_launch(c, w, ws, n, tokens, 0, st))) return rc;
  if (timed) KX_HIP(hipEventRecord(ws->ev[2], st));
  // shared down + combine + residual: as the epilogue of a GEMV of its own, or, for one token, inside the routed
  // down launch (whichever workgroup completes a block of rows combines it)
  KxGemvArgs d = {};
  d.w0 = (const uint16_t *)w->d_shared_down; d.x = ws->smid; d.x_stride = c->shared_inter; d.out = d_x;
  d.out_stride = H; d.rows = H; d.cols = c->shared_inter; d.tokens = tokens; d.expert_out = ws->eout;
  d.route_w = ws->weights; d.topk = K; d.flags = flags & 1u;
  bool tailed = false;
  if (paired && tokens == 1 && !(flags & KX_MOE_SEPARATE_TAIL) && H / 16 <= KX_TAIL_BLOCKS) {
    KxMoeTail t = {};
    t.counter = ws->tail_count; t.n_active = ws->n_active; t.sy = ws->sy; t.route_w = ws->weights; t.x = (uint16_t *)d_x;
    t.x_stride = H; t.tokens = tokens; t.topk = K; t.flags = flags & 1u;
    const int I = c->moe_inter;
    if ((rc = kx_i4_down_shared_launch((const uint32_t *)w->d_down_packed, (const uint16_t *)w->d_down_scale, ws->mid, ws->eout,
                                       ws->work, ws->pairs, H, I, 1, (size_t)H * (I / 8), (size_t)H * (I / 32),
                                       (long)tokens * K < E ? tokens * K : E, d, t, &tailed, st))) return rc;
  }
  // routed down
  if (rmm) {
    const int I = c->moe_inter;
    bool mm_done = false;
    if (i4mm &&
        (rc = kx_i4mm_launch(false, (const uint32_t *)w->d_down_packed, (const uint16_t *)w->d_down_scale, nullptr, nullptr, ws->mid,
                             ws->eout, ws->work, ws->pairs, n_slots, H, I, 1, (size_t)H * (I / 8), (size_t)H * (I / 32), rmm_min,
                             1 << 30, kx_cdiv(tokens, 32), &mm_done, st))) return rc;
    if (!mm_done &&
        (rc = kx_grouped_gemm_launch(false, true, w->d_down_packed, (const uint16_t *)w->d_down_scale, nullptr, nullptr,
                                     ws->mid, ws->eout, KX_GG_BF16, ws->work, ws->pairs, 0, n_slots, H, I, 1, (size_t)H * (I / 8),
                                     (size_t)H * (I / 32), tokens, st, rmm_min))) return rc;
    if ((rc = kx_i4_launch(false, (const uint32_t *)w->d_down_packed, (const uint16_t *)w->d_down_scale, nullptr, nullptr,
                           ws->mid, ws->eout, ws->work, ws->pairs, 0, H, I, 1, (size_t)H * (I / 8), (size_t)H * (I / 32),
                           1, n_slots, 1, rmm_min - 1, ws->side, 2))) return rc;
  } else if (!tailed && (rc = routed_launch(c, w, ws, n, tokens, 1, st))) return rc;
  if (timed) KX_HIP(hipEventRecord(ws->ev[3], st));
  // shared gate/up + SwiGLU when it neither rode with the router nor ran on the side stream
  if (!paired && !shared_up_done) {
    if (norm_w) { s.x = n; s.norm_w = nullptr; }  // d_n holds the normed rows by now
    if ((rc = kx_gemv_launch(KX_EPI_SWIGLU, s, st))) return rc;
  }
  if (timed) KX_HIP(hipEventRecord(ws->ev[4], st));
  if (!tailed) {
    if (forked) {  // the GEMV class of the routed experts and the shared expert are in before anything reads their outputs
      KX_HIP(hipEventRecord(ws->join, ws->side));
      KX_HIP(hipStreamWaitEvent(st, ws->join, 0));
    }
    if (shared_down_done) {  // the shared output is in sy: the combine is a kernel of its own
      if ((rc = kx_moe_combine_launch(ws->eout, ws->weights, ws->sy, (uint16_t *)d_x, tokens, H, K, flags & 1u, st))) return rc;
    } else if ((rc = kx_gemv_launch(KX_EPI_MOE_COMBINE, d, st))) return rc;
  }
  if (timed) KX_HIP(hipEventRecord(ws->ev[5], st));
  return KX_OK;
}

extern "C" int kx_moe_decode_layer(const kx_config *cfg, const kx_moe_weights *w, kx_moe_workspace *ws, const void *d_n,
                                   void *d_x, int32_t tokens, uint32_t flags, void *stream) {
  return kx_moe_layer_launch(cfg, w, ws, (void *)d_n, d_x, tokens, flags & KX_MOE_PUBLIC_FLAGS, nullptr, kx_stream(stream), false);
}

extern "C" int kx_moe_decode_layer_timed(const kx_config *cfg, const kx_moe_weights *w, kx_moe_workspace *ws,
                                         const void *d_n, void *d_x, int32_t tokens, uint32_t flags, void *stream,
                                         float *ms5) {
  KX_REQUIRE(ms5, "kx_moe_decode_layer_timed: null output");
  int rc = kx_moe_layer_launch(cfg, w, ws, (void *)d_n, d_x, tokens, flags & KX_MOE_PUBLIC_FLAGS, nullptr, kx_stream(stream), true);
  if (rc) return rc;
  KX_HIP(hipEventSynchronize(ws->ev[5]));
  for (int i = 0; i < 5; ++i) KX_HIP(hipEventElapsedTime(&ms5[i], ws->ev[i], ws->ev[i + 1]));
  return KX_OK;
}

// One routed-expert kernel alone, on the routing the most recent decode-layer call left in the workspace
// (for timing the kernel back to back): which = 0 gate/up + SwiGLU (d_n -> mid), 1 down (mid -> expert outputs).
extern "C" int kx_moe_routed_only(const kx_config *c, const kx_moe_weights *w, kx_moe_workspace *ws, const void *d_n,
                                  int32_t tokens, int32_t which, void *stream) {
  int rc = check_cfg(c);
  if (rc) return rc;
  KX_REQUIRE(w && ws && d_n, "kx_moe_routed_only: null argument");
  KX_REQUIRE(tokens > 0 && tokens <= ws->max_tokens, "kx_moe_routed_only: tokens=%d outside [1, %d]", tokens, ws->max_tokens);
  KX_REQUIRE(which == 0 || which == 1, "kx_moe_routed_only: which=%d", which);
  return routed_launch(c, w, ws, (const uint16_t *)d_n, tokens, which, kx_stream(stream));
}

// ---- prefill chunk through one MoE layer: grouped GEMMs on the matrix cores ------------------
extern "C" int kx_moe_prefill_layer(const kx_config *c, const kx_moe_weights *w, kx_moe_workspace *ws, const void *d_n,
                                    void *d_x, int32_t tokens, uint32_t flags, void *stream) {
  int rc = check_cfg(c);
  if (rc) return rc;
  KX_REQUIRE(w && ws && d_n && d_x, "kx_moe_prefill_layer: null argument");
  KX_REQUIRE(tokens > 0 && tokens <= ws->max_tokens, "kx_moe_prefill_layer: tokens=%d outside [1, %d]", tokens, ws->max_tokens);
  KX_REQUIRE(c->hidden == ws->cfg.hidden && c->moe_inter == ws->cfg.moe_inter && c->experts == ws->cfg.experts &&
                 c->topk == ws->cfg.topk && c->shared_inter == ws->cfg.shared_inter,
             "kx_moe_prefill_layer: workspace was created for another shape");
  hipStream_t st = kx_stream(stream);
  const int H = c->hidden, I = c->moe_inter, SI = c->shared_inter, E = c->experts, K = c->topk;
  const uint16_t *n = (const uint16_t *)d_n;
  // The shared expert needs nothing from the router or the routed experts: its two GEMMs run on the side stream
  // while this one routes and runs the grouped GEMMs, and are joined before the combine.
  KX_HIP(hipEventRecord(ws->fork, st));
  KX_HIP(hipStreamWaitEvent(ws->side, ws->fork, 0));
  if ((rc = kx_grouped_gemm_launch(true, false, w->d_shared_gate, nullptr, w->d_shared_up, nullptr, n, ws->smid, KX_GG_BF16,
                                   nullptr, nullptr, tokens, 1, SI, H, 1, 0, 0, tokens, ws->side))) return rc;
  if ((rc = kx_grouped_gemm_launch(false, false, w->d_shared_down, nullptr, nullptr, nullptr, ws->smid, ws->sy, KX_GG_BF16,
                                   nullptr, nullptr, tokens, 1, H, SI, 1, 0, 0, tokens, ws->side))) return rc;
  KX_HIP(hipEventRecord(ws->join, ws->side));
  // router: fp32 logits (unrounded) as one GEMM of all tokens against the gate, top-k, bucketing.  Up to 32 tokens
  // the decode GEMV is used instead (its summation order is the decode path's).
  if (tokens <= 32) {
    KxGemvArgs g = {};
    g.w0 = (const uint16_t *)w->d_router_gate; g.x = n; g.x_stride = H; g.out = ws->logits; g.out_stride = E;
    g.rows = E; g.cols = H; g.tokens = tokens;
    if ((rc = kx_gemv_launch(KX_EPI_F32, g, st))) return rc;
  } else {
    if ((rc = kx_grouped_gemm_launch(false, false, w->d_router_gate, nullptr, nullptr, nullptr, n, ws->logits, KX_GG_F32, nullptr,
                                     nullptr, tokens, 1, E, H, 1, 0, 0, tokens, st))) return rc;
  }
  if ((rc = kx_router_topk_launch(ws->logits, (const float *)w->d_router_bias, ws->ids, ws->weights, tokens, E, K,
                                  c->routed_scale, st))) return rc;
  if ((rc = kx_bucket_launch(ws->ids, tokens, E, K, ws->counts, ws->offsets, ws->pairs, ws->work, ws->n_active, st)))
    return rc;
  const int n_slots = (long)tokens * K < E ? tokens * K : E;
  // routed experts: gate/up + SwiGLU, then down
  if ((rc = kx_grouped_gemm_launch(true, true, w->d_gate_packed, (const uint16_t *)w->d_gate_scale, w->d_up_packed,
                                   (const uint16_t *)w->d_up_scale, n, ws->mid, KX_GG_BF16, ws->work, ws->pairs, 0, n_slots, I, H,
                                   K, (size_t)I * (H / 8), (size_t)I * (H / 32), tokens, st))) return rc;
  if ((rc = kx_grouped_gemm_launch(false, true, w->d_down_packed, (const uint16_t *)w->d_down_scale, nullptr, nullptr,
                                   ws->mid, ws->eout, KX_GG_BF16, ws->work, ws->pairs, 0, n_slots, H, I, 1, (size_t)H * (I / 8),
                                   (size_t)H * (I / 32), tokens, st))) return rc;
  KX_HIP(hipStreamWaitEvent(st, ws->join, 0));  // the shared expert's output
  return kx_moe_combine_launch(ws->eout, ws->weights, ws->sy, (uint16_t *)d_x, tokens, H, K, flags, st);
}
