// kx_model.hip -- the decoder stack: prefill, decode step, greedy sample, generate.
//
// Reference: generate() and its run() lambda, src/kimi_exec.cu:780-893.  The
// reference allocates 19 single-token fp32 scratch buffers (:792-799), streams
// every weight tile from NVMe inside the layer loop and synchronises with the
// host once per MoE layer (:844) and twice per vocabulary tile (:728-730).
// Here one arena in HBM holds the weights (seeded random-init, kx_model_create, or
// copied in from the checkpoint a runtime-index.blok describes, kx_model_load), the latent KV
// cache and the scratch of a step for `max_batch` sequences; a step enqueues
// kernels on one stream and never waits for the host.
//
// Per layer (T = batch tokens, all at the same position; up to 4 tokens the RMSNorms run in the
// prologue of the GEMV that consumes them):
//   [q_a ; kv_a] GEMV (input norm) -> q_b GEMV (q_a norm) -> W_UK absorb + rope(q), with one
//   workgroup that norms kv_a, rotates the rope key and writes the cache row -> attention
//   partials over the latent cache -> W_UV GEMV per head (merges the partials as it loads
//   them) -> o_proj GEMV with the residual add
//   -> dense SwiGLU MLP (layers < first_dense) or the routed MoE layer (post-attention norm
//   in their first GEMV).
// From 5 sequences on the dense projections run as GEMMs on the matrix cores.
#include <math.h>
#include <string.h>
#include <vector>
#include "kx_attn_parts.h"
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_front.h"
#include "kx_index.h"
#include "kx_load.h"
#include "kx_mla.h"

namespace {

enum {  // tensor ids: global tensors use the id itself, layer L uses (L+1)*64 + id
  TID_EMBED = 1, TID_FINAL_NORM = 2, TID_LM_HEAD = 3,
  TL_INPUT_LN = 0, TL_QA = 1, TL_QA_LN = 2, TL_QB = 3, TL_KVA = 4, TL_KV_LN = 5, TL_KVB = 6, TL_O = 7, TL_POST_LN = 8,
  TL_DENSE_GATE = 9, TL_DENSE_UP = 10, TL_DENSE_DOWN = 11, TL_ROUTER = 12, TL_ROUTER_BIAS = 13,
  TL_GATE_P = 14, TL_GATE_S = 15, TL_UP_P = 16, TL_UP_S = 17, TL_DOWN_P = 18, TL_DOWN_S = 19,
  TL_SH_GATE = 20, TL_SH_UP = 21, TL_SH_DOWN = 22
};

struct Layer {
  uint16_t *input_ln, *qkv_a, *qa_ln, *qb, *kv_ln, *kvb, *o, *post_ln;
  uint16_t *dgate, *dup, *ddown;
  kx_moe_weights moe;
  uint16_t *cache;  // [max_batch][max_context][kv_rank + qk_rope]
};

__global__ void embed_k(const uint16_t *__restrict__ embed, const uint32_t *__restrict__ ids, uint16_t *__restrict__ x,
                        int hidden) {
  const uint4 *src = (const uint4 *)(embed + (size_t)ids[blockIdx.x] * hidden);
  uint4 *dst = (uint4 *)(x + (size_t)blockIdx.x * hidden);
  for (int i = threadIdx.x; i < hidden / 8; i += blockDim.x) dst[i] = src[i];
}
// the per-head W_UV products of a long prefill step as one grouped GEMM: group h = the rows t * heads + h of the
// [tokens * heads, kv_rank] view of the attention output, in token order
__global__ void head_groups_k(int tokens, int heads, int4 *__restrict__ work, int *__restrict__ pairs) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= tokens * heads) return;
  const int h = idx / tokens, t = idx - h * tokens;
  pairs[idx] = t * heads + h;
  if (t == 0) work[h] = make_int4(h, h * tokens, (h + 1) * tokens, h);
}
__global__ void copy_ids_k(const uint32_t *__restrict__ src, uint32_t *__restrict__ dst, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

}  // namespace

struct kx_model {
  kx_config c;
  char *arena = nullptr;
  size_t arena_bytes = 0;
  uint16_t *embed, *final_norm, *lm_head, *rope_tab;
  std::vector<Layer> layers;
  // scratch of one step
  uint16_t *x, *n, *qkv, *qa, *q, *o_lat, *att, *dmid;
  float *qabs, *partial, *logits, *argmax_scratch;
  uint32_t *ids, *next, *history;  // [max_context][B], [B], [max_context][B]
  int *head_count;                 // [heads] arrival counters of the q_b GEMV that finishes the query; zero between launches
  int *hand_err;                   // error flag of the resident launches (kx_front.hip, kx_i4.hip): a wait for another workgroup's values gave up
  uint32_t *front_hand;            // tagged words of the attention block's front launch (q_a, kv_a, q)
  uint32_t front_tag = 0;          // tag of its last launch
  uint32_t *back_hand;             // tagged words of the attention block's back launch (attention output, residual row, router logits)
  uint32_t back_tag = 0;
  int4 *head_work;                 // [heads], [step tokens * heads]: the groups of head_groups_k
  int *head_pairs;
  uint32_t fusion = KX_FUSE_ALL;
  int mla_kernel = KX_MLA_AUTO;    // kx_model_set_attention_kernel
  float *route_logits = nullptr;   // routing record (kx_model_set_routing_record): [n_layers][max_batch][experts]
  int *route_distinct = nullptr;   // [n_layers] distinct experts of the last step
  float *route_history = nullptr;  // record level 2: router logits of every position, [n_layers][max_context][max_batch][experts]
  kx_moe_workspace *moe_ws = nullptr;
  hipStream_t st = nullptr;
  hipEvent_t ev[3] = {nullptr, nullptr, nullptr};
  int batch = 0, pos = 0;
  int prefill_chunk = 1;  // prompt positions per prefill step (kx_model_set_prefill_chunk)
  uint32_t exact = 0;     // kx_model_set_exact: KX_EXACT_* parts that keep the bit-reproducible kernels at every batch size
  int x_row0 = 0;         // first row of x that belongs to the last position of the last step
  bool sampled = false;
  float ms_prefill = 0, ms_decode = 0;
  int steps_decoded = 0;  // ids sampled per sequence by the last kx_generate (less than asked for when every sequence ended)
  uint64_t load_bytes = 0;  // checkpoint bytes copied in by kx_model_load, and the time that took
  double load_seconds = 0;
};

namespace {

// tokens a step may carry: a decode step has one per sequence, a prefill step up to this many (positions x sequences)
constexpr int STEP_TOKENS = 2048;
inline int step_tokens(const kx_config *c) { return c->max_batch > STEP_TOKENS ? c->max_batch : STEP_TOKENS; }
// entries (position x sequence) one attention launch of a prefill step takes; the partials are laid out for these
constexpr int ATT_ENTRIES = 256;
inline int att_entries(const kx_config *c) { return c->max_batch > ATT_ENTRIES ? c->max_batch : ATT_ENTRIES; }

struct Plan {  // byte offsets of everything in the arena
  size_t total = 0, weights = 0, cache = 0, scratch = 0;
  size_t take(size_t bytes) {
    size_t at = total;
    total += (bytes + 255) & ~(size_t)255;
    return at;
  }
};

int check_model_cfg(const kx_config *c) {
  KX_REQUIRE(c, "kx_model: null config");
  KX_REQUIRE(c->n_layers > 0 && c->first_dense >= 0 && c->first_dense <= c->n_layers, "kx_model: n_layers=%d first_dense=%d", c->n_layers, c->first_dense);
  KX_REQUIRE(c->hidden > 0 && c->hidden % 1024 == 0, "kx_model: hidden=%d must be a multiple of 1024", c->hidden);
  KX_REQUIRE(c->q_rank > 0 && c->q_rank % 512 == 0, "kx_model: q_rank=%d must be a multiple of 512", c->q_rank);
  KX_REQUIRE(c->kv_rank == 512 && c->qk_rope == 64, "kx_model: kv_rank=%d qk_rope=%d must be 512 and 64", c->kv_rank, c->qk_rope);
  KX_REQUIRE(c->heads > 0 && c->heads % 4 == 0, "kx_model: heads=%d must be a multiple of 4", c->heads);
  KX_REQUIRE(c->qk_nope > 0 && c->qk_nope % 8 == 0 && c->v_head > 0 && (c->heads * c->v_head) % 512 == 0,
             "kx_model: qk_nope=%d v_head=%d", c->qk_nope, c->v_head);
  KX_REQUIRE(c->first_dense == 0 || (c->dense_inter > 0 && c->dense_inter % 512 == 0), "kx_model: dense_inter=%d must be a multiple of 512", c->dense_inter);
  KX_REQUIRE(c->vocab > 0 && c->max_batch > 0 && c->max_context > 0, "kx_model: vocab=%d max_batch=%d max_context=%d", c->vocab, c->max_batch, c->max_context);
  if (c->first_dense < c->n_layers) {
    KX_REQUIRE(c->moe_inter > 0 && c->moe_inter % 1024 == 0, "kx_model: moe_inter=%d must be a multiple of 1024", c->moe_inter);
    KX_REQUIRE(c->shared_inter > 0 && c->shared_inter % 512 == 0, "kx_model: shared_inter=%d must be a multiple of 512", c->shared_inter);
    KX_REQUIRE(c->experts > 0 && c->experts <= 1024 && c->topk > 0 && c->topk <= c->experts, "kx_model: experts=%d topk=%d", c->experts, c->topk);
  }
  return KX_OK;
}

// lays the model out; when m != nullptr also sets its pointers (arena must be allocated)
int layout(const kx_config *c, Plan &p, kx_model *m) {
  const size_t H = c->hidden, V = c->vocab, E = c->experts, I = c->moe_inter, SI = c->shared_inter, D = c->dense_inter;
  const size_t KD = (size_t)c->heads * (c->qk_nope + c->qk_rope), VD = (size_t)c->heads * c->v_head;
  const size_t KVA = c->kv_rank + c->qk_rope, KVB = (size_t)c->heads * (c->qk_nope + c->v_head), B = c->max_batch;
  char *base = m ? m->arena : nullptr;
#define KX_AT(T, bytes) ((T)(base + p.take(bytes)))
  auto *embed = KX_AT(uint16_t *, V * H * 2);
  auto *final_norm = KX_AT(uint16_t *, H * 2);
  auto *lm_head = KX_AT(uint16_t *, V * H * 2);
  auto *rope_tab = KX_AT(uint16_t *, (size_t)c->max_context * c->qk_rope * 2);
  if (m) { m->embed = embed; m->final_norm = final_norm; m->lm_head = lm_head; m->rope_tab = rope_tab; m->layers.resize(c->n_layers); }
  for (int l = 0; l < c->n_layers; ++l) {
    Layer L = {};
    L.input_ln = KX_AT(uint16_t *, H * 2);
    L.qkv_a = KX_AT(uint16_t *, ((size_t)c->q_rank + KVA) * H * 2);
    L.qa_ln = KX_AT(uint16_t *, (size_t)c->q_rank * 2);
    L.qb = KX_AT(uint16_t *, KD * c->q_rank * 2);
    L.kv_ln = KX_AT(uint16_t *, (size_t)c->kv_rank * 2);
    L.kvb = KX_AT(uint16_t *, KVB * c->kv_rank * 2);
    L.o = KX_AT(uint16_t *, H * VD * 2);
    L.post_ln = KX_AT(uint16_t *, H * 2);
    if (l < c->first_dense) {
      L.dgate = KX_AT(uint16_t *, D * H * 2);
      L.dup = KX_AT(uint16_t *, D * H * 2);
      L.ddown = KX_AT(uint16_t *, H * D * 2);
    } else {
      L.moe.d_router_gate = KX_AT(void *, E * H * 2);
      L.moe.d_router_bias = KX_AT(void *, E * 4);
      L.moe.d_gate_packed = KX_AT(void *, E * I * H / 2);
      L.moe.d_gate_scale = KX_AT(void *, E * I * H / 32 * 2);
      L.moe.d_up_packed = KX_AT(void *, E * I * H / 2);
      L.moe.d_up_scale = KX_AT(void *, E * I * H / 32 * 2);
      L.moe.d_down_packed = KX_AT(void *, E * H * I / 2);
      L.moe.d_down_scale = KX_AT(void *, E * H * I / 32 * 2);
      L.moe.d_shared_gate = KX_AT(void *, SI * H * 2);
      L.moe.d_shared_up = KX_AT(void *, SI * H * 2);
      L.moe.d_shared_down = KX_AT(void *, H * SI * 2);
    }
    if (m) m->layers[l] = L;
  }
  p.weights = p.total;
  for (int l = 0; l < c->n_layers; ++l) {
    auto *cache = KX_AT(uint16_t *, B * c->max_context * KVA * 2);
    if (m) m->layers[l].cache = cache;
  }
  p.cache = p.total - p.weights;
  const size_t inter = D > KD ? D : KD;
  const size_t BT = step_tokens(c);  // rows of the per-token scratch
  auto *x = KX_AT(uint16_t *, BT * H * 2);
  auto *n = KX_AT(uint16_t *, BT * H * 2);
  auto *qkv = KX_AT(uint16_t *, BT * ((size_t)c->q_rank + KVA) * 2);
  auto *qa = KX_AT(uint16_t *, BT * (size_t)c->q_rank * 2);
  auto *q = KX_AT(uint16_t *, BT * KD * 2);
  auto *o_lat = KX_AT(uint16_t *, BT * (size_t)c->heads * c->kv_rank * 2);
  auto *att = KX_AT(uint16_t *, BT * VD * 2);
  auto *dmid = KX_AT(uint16_t *, BT * inter * 2);
  auto *qabs = KX_AT(float *, BT * (size_t)c->heads * KVA * 4);
  auto *partial = KX_AT(float *, kx_mla_partial_floats(att_entries(c), c->heads, c->kv_rank, c->max_context) * 4);
  auto *logits = KX_AT(float *, B * V * 4);
  auto *argmax_scratch = KX_AT(float *, KX_ARGMAX_SCRATCH_FLOATS(B) * 4);
  auto *ids = KX_AT(uint32_t *, (size_t)c->max_context * B * 4);
  auto *next = KX_AT(uint32_t *, B * 4);
  auto *history = KX_AT(uint32_t *, (size_t)c->max_context * B * 4);
  auto *head_count = KX_AT(int *, (size_t)c->heads * 4);
  auto *hand_err = KX_AT(int *, 4);
  auto *front_hand = KX_AT(uint32_t *, kx_front_hand_words(c->q_rank, (int)KVA, (int)KD) * 4);
  auto *back_hand = KX_AT(uint32_t *, kx_back_hand_words((int)VD, c->hidden, c->experts) * 4);
  auto *head_work = KX_AT(int4 *, (size_t)c->heads * 16);
  auto *head_pairs = KX_AT(int *, BT * c->heads * 4);
#undef KX_AT
  p.scratch = p.total - p.weights - p.cache;
  if (m) {
    m->x = x; m->n = n; m->qkv = qkv; m->qa = qa; m->q = q; m->o_lat = o_lat; m->att = att; m->dmid = dmid;
    m->qabs = qabs; m->partial = partial; m->logits = logits; m->argmax_scratch = argmax_scratch; m->ids = ids; m->next = next; m->history = history;
    m->head_count = head_count; m->hand_err = hand_err; m->front_hand = front_hand; m->back_hand = back_hand; m->head_work = head_work; m->head_pairs = head_pairs;
  }
  return KX_OK;
}

// rope table for every position, computed on the host
int init_rope(kx_model *m) {
  const kx_config &c = m->c;
  std::vector<uint16_t> tab((size_t)c.max_context * c.qk_rope);
  int rc = kx_rope_table(&c, 0, c.max_context, tab.data());
  if (rc) return rc;
  KX_HIP(hipMemcpyAsync(m->rope_tab, tab.data(), tab.size() * 2, hipMemcpyHostToDevice, m->st));
  KX_HIP(hipStreamSynchronize(m->st));
  return KX_OK;
}

int init_weights(kx_model *m) {
  const kx_config &c = m->c;
  const size_t H = c.hidden, V = c.vocab, E = c.experts, I = c.moe_inter, SI = c.shared_inter, D = c.dense_inter;
  const size_t KD = (size_t)c.heads * (c.qk_nope + c.qk_rope), VD = (size_t)c.heads * c.v_head;
  const size_t KVA = c.kv_rank + c.qk_rope, KVB = (size_t)c.heads * (c.qk_nope + c.v_head);
  const float sg = c.init_sigma, es = c.expert_scale_sigma;
  void *st = m->st;
  int rc;
#define KX_TRY(call) do { if ((rc = (call))) return rc; } while (0)
  KX_TRY(kx_fill_normal_bf16(m->embed, V * H, c.seed, TID_EMBED, 1.0f, 0, st));
  KX_TRY(kx_fill_affine_bf16(m->final_norm, H, c.seed, TID_FINAL_NORM, 1.0f, 0.02f, st));
  KX_TRY(kx_fill_normal_bf16(m->lm_head, V * H, c.seed, TID_LM_HEAD, sg, 0, st));
  for (int l = 0; l < c.n_layers; ++l) {
    Layer &L = m->layers[l];
    const uint64_t b = (uint64_t)(l + 1) * 64;
    KX_TRY(kx_fill_affine_bf16(L.input_ln, H, c.seed, b + TL_INPUT_LN, 1.0f, 0.02f, st));
    KX_TRY(kx_fill_normal_bf16(L.qkv_a, (size_t)c.q_rank * H, c.seed, b + TL_QA, sg, 0, st));
    KX_TRY(kx_fill_normal_bf16(L.qkv_a + (size_t)c.q_rank * H, KVA * H, c.seed, b + TL_KVA, sg, 0, st));
    KX_TRY(kx_fill_affine_bf16(L.qa_ln, c.q_rank, c.seed, b + TL_QA_LN, 1.0f, 0.02f, st));
    KX_TRY(kx_fill_normal_bf16(L.qb, KD * c.q_rank, c.seed, b + TL_QB, sg, 0, st));
    KX_TRY(kx_fill_affine_bf16(L.kv_ln, c.kv_rank, c.seed, b + TL_KV_LN, 1.0f, 0.02f, st));
    KX_TRY(kx_fill_normal_bf16(L.kvb, KVB * c.kv_rank, c.seed, b + TL_KVB, sg, 0, st));
    KX_TRY(kx_fill_normal_bf16(L.o, H * VD, c.seed, b + TL_O, sg, 0, st));
    KX_TRY(kx_fill_affine_bf16(L.post_ln, H, c.seed, b + TL_POST_LN, 1.0f, 0.02f, st));
    if (l < c.first_dense) {
      KX_TRY(kx_fill_normal_bf16(L.dgate, D * H, c.seed, b + TL_DENSE_GATE, sg, 0, st));
      KX_TRY(kx_fill_normal_bf16(L.dup, D * H, c.seed, b + TL_DENSE_UP, sg, 0, st));
      KX_TRY(kx_fill_normal_bf16(L.ddown, H * D, c.seed, b + TL_DENSE_DOWN, sg, 0, st));
    } else {
      kx_moe_weights &w = L.moe;
      KX_TRY(kx_fill_normal_bf16((void *)w.d_router_gate, E * H, c.seed, b + TL_ROUTER, 1.0f / sqrtf((float)H), 0, st));
      KX_TRY(kx_fill_normal_f32((void *)w.d_router_bias, E, c.seed, b + TL_ROUTER_BIAS, 0.01f, st));
      KX_TRY(kx_fill_words_u32((void *)w.d_gate_packed, E * I * H / 8, c.seed, b + TL_GATE_P, st));
      KX_TRY(kx_fill_normal_bf16((void *)w.d_gate_scale, E * I * H / 32, c.seed, b + TL_GATE_S, es, 1, st));
      KX_TRY(kx_fill_words_u32((void *)w.d_up_packed, E * I * H / 8, c.seed, b + TL_UP_P, st));
      KX_TRY(kx_fill_normal_bf16((void *)w.d_up_scale, E * I * H / 32, c.seed, b + TL_UP_S, es, 1, st));
      KX_TRY(kx_fill_words_u32((void *)w.d_down_packed, E * H * I / 8, c.seed, b + TL_DOWN_P, st));
      KX_TRY(kx_fill_normal_bf16((void *)w.d_down_scale, E * H * I / 32, c.seed, b + TL_DOWN_S, es, 1, st));
      KX_TRY(kx_fill_normal_bf16((void *)w.d_shared_gate, SI * H, c.seed, b + TL_SH_GATE, sg, 0, st));
      KX_TRY(kx_fill_normal_bf16((void *)w.d_shared_up, SI * H, c.seed, b + TL_SH_UP, sg, 0, st));
      KX_TRY(kx_fill_normal_bf16((void *)w.d_shared_down, H * SI, c.seed, b + TL_SH_DOWN, sg, 0, st));
    }
  }
#undef KX_TRY
  return init_rope(m);
}

// one run() of the reference for `B` tokens at position m->pos; ids on the device.
// C > 1 (prefill): C consecutive positions of every sequence in one step, tokens position-major (token i * B + b is
// position pos + i of sequence b).  Everything but the attention is per token, so the step runs as a batch of B * C
// tokens; the q absorb writes the cache rows of all C positions, then position i attends to rows 0 .. pos + i (one
// launch each, the kernels take the position from the token index).  Only the last position is sampled.
int step(kx_model *m, const uint32_t *d_ids, bool sample, int C = 1) {
  const kx_config &c = m->c;
  const int NB = m->batch, B = NB * C, H = c.hidden, pos = m->pos;
  const int KD = c.heads * (c.qk_nope + c.qk_rope), VD = c.heads * c.v_head, KVA = c.kv_rank + c.qk_rope;
  const int QKV = c.q_rank + KVA;
  hipStream_t st = m->st;
  int rc;
#define KX_TRY(call) do { if ((rc = (call))) return rc; } while (0)
  hipLaunchKernelGGL(embed_k, dim3(B), dim3(256), 0, st, m->embed, d_ids, m->x, H);  // embed_token (:651-655)
  KX_LAUNCH_CHECK();
  const uint16_t *rope_row = m->rope_tab + (size_t)pos * c.qk_rope;
  const size_t seq_stride = (size_t)c.max_context * KVA;
  const bool fuse = B <= 4 && C == 1;  // RMSNorms ride in the prologue of the GEMV that consumes them
  // From 5 sequences on (the fused prologues cover up to 4), the dense projections run as GEMMs on the matrix cores: the
  // GEMV is bound by its fma count there.  Same values, another summation order (the bf16 rounding points stay).
  const bool mm = B >= 5 && !(m->exact & KX_EXACT_PROJECTIONS);
  const int mla_kernel = (m->exact & KX_EXACT_ATTENTION) ? KX_MLA_VALU : m->mla_kernel;
  auto dense = [&](int epi, const KxGemvArgs &g) -> int {
    if (!mm) return kx_gemv_launch(epi, g, st);
    const bool dual = epi == KX_EPI_SWIGLU;
    const int mode = epi == KX_EPI_RESID ? KX_GG_RESID : epi == KX_EPI_ARGMAX ? KX_GG_F32_OF_BF16 : epi == KX_EPI_F32 ? KX_GG_F32 : KX_GG_BF16;
    if (g.tokens <= 32) {  // one tile: the kernel built for it
      bool done = false;
      int rc2 = kx_skinny_gemm_launch(dual, g.w0, dual ? g.w1 : nullptr, g.x, g.x_stride, g.out, g.out_stride, mode, g.tokens, g.rows,
                                      g.cols, &done, st);
      if (rc2 || done) return rc2;
    }
    KX_REQUIRE(g.x_stride == g.cols && g.out_stride == g.rows, "kx_model: the GEMM kernel takes dense activation and output rows");
    return kx_grouped_gemm_launch(dual, false, g.w0, nullptr, dual ? g.w1 : nullptr, nullptr, g.x, g.out, mode, nullptr, nullptr,
                                  g.tokens, 1, g.rows, g.cols, 1, 0, 0, g.tokens, st);
  };
  for (int l = 0; l < c.n_layers; ++l) {
    bool moe_head_done = false;  // the MoE layer's router + shared gate/up step rode in the attention block's last launch
    Layer &L = m->layers[l];
    KxGemvArgs g = {};
    g.w0 = L.qkv_a; g.x = m->n; g.x_stride = H; g.out = m->qkv; g.out_stride = QKV; g.rows = QKV; g.cols = H; g.tokens = B;
    if (fuse) { g.x = m->x; g.norm_w = L.input_ln; g.norm_eps = c.rms_eps; }
    KxGemvArgs gb = {};
    gb.w0 = L.qb; gb.x = m->qa; gb.x_stride = c.q_rank; gb.out = m->q; gb.out_stride = KD; gb.rows = KD; gb.cols = c.q_rank; gb.tokens = B;
    if (fuse) { gb.x = m->qkv; gb.x_stride = QKV; gb.norm_w = L.qa_ln; gb.norm_eps = c.rms_eps; }
    QAbsArgs qa = {};
    qa.q = m->q; qa.kvb = L.kvb; qa.rope_row = rope_row; qa.qabs = m->qabs; qa.kva = m->qkv + c.q_rank; qa.kva_stride = QKV;
    qa.w_kv_ln = L.kv_ln; qa.cache = L.cache; qa.seq_stride = seq_stride; qa.heads = c.heads; qa.nope = c.qk_nope;
    qa.rope = c.qk_rope; qa.v_head = c.v_head; qa.kv_rank = c.kv_rank; qa.pos = pos; qa.eps = c.rms_eps;
    qa.head_count = m->head_count;
    // One token: the whole front of the attention block -- q_a | kv_a, q_b, the W_UK absorb, RoPE, the cache row -- as
    // one resident launch where the shapes and the device allow it (kx_front.hip; same sums, same bits)
    bool front = false;
    if (fuse && B == 1 && (m->fusion & KX_FUSE_FRONT)) {
      const uint32_t tag = m->front_tag % 65535u + 1u;
      KX_TRY(kx_attn_front_launch(g, gb, qa, m->front_hand, tag, m->hand_err, &front, st));
      if (front) m->front_tag = tag;
    }
    if (!front) {
      if (!fuse) KX_TRY(kx_rmsnorm_launch(m->x, L.input_ln, m->n, B, H, H, H, c.rms_eps, st));                 // :812
      KX_TRY(dense(KX_EPI_BF16, g));                                                                      // :813, :816
      if (!fuse) KX_TRY(kx_rmsnorm_launch(m->qkv, L.qa_ln, m->qa, B, c.q_rank, QKV, c.q_rank, c.rms_eps, st)); // :814
      // W_UK absorb + rope(q); kv_a norm, rope of the shared key, cache row (:817-824): inside the q_b launch when
      // the shapes allow, else as a kernel of their own
      bool absorbed = false;
      if (fuse && (m->fusion & KX_FUSE_ABSORB)) KX_TRY(kx_gemv_absorb_launch(gb, qa, &absorbed, st));     // :815
      if (!absorbed) {
        KX_TRY(dense(KX_EPI_BF16, gb));                                                                   // :815
        KX_TRY(kx_q_absorb_launch(m->q, L.kvb, rope_row, m->qabs, B, c.heads, c.qk_nope, c.qk_rope, c.v_head, c.kv_rank,
                                  m->qkv + c.q_rank, QKV, L.kv_ln, L.cache, seq_stride, pos, c.rms_eps, st, C > 1 ? NB : 0));
      }
    }
    g = {};  // W_UV of :818 per head
    g.w0 = L.kvb; g.x = m->o_lat; g.x_stride = c.heads * c.kv_rank; g.out = m->att; g.out_stride = VD; g.rows = VD;
    g.cols = c.kv_rank; g.tokens = B; g.row_block = c.v_head; g.w_block_stride = c.qk_nope + c.v_head;
    g.w_block_off = c.qk_nope; g.x_block_stride = c.kv_rank;
    if (fuse) {                                                                                 // :825
      KxMlaPartials mp;
      KX_TRY(kx_mla_partials_launch(&c, L.cache, seq_stride, m->qabs, m->partial, B, pos + 1, &mp, st, 0, mla_kernel));
      if (mp.spans <= 64) {  // the GEMV's activations are the attention partials, merged as they are loaded
        g.mla_pm = mp.pm; g.mla_pz = mp.pz; g.mla_po = mp.po; g.mla_spans = mp.spans; g.mla_heads = c.heads;
      } else {               // long context, few sequences: more spans than the GEMV's merge takes
        KX_TRY(kx_mla_combine_launch(mp, m->o_lat, B, c.heads, st));
      }
    } else {
      // at most ATT_ENTRIES entries a launch: whole positions, in order
      const int cs = NB >= ATT_ENTRIES ? 1 : ATT_ENTRIES / NB;
      for (int i0 = 0; i0 < C; i0 += cs) {
        const int np = C - i0 < cs ? C - i0 : cs;
        KX_TRY(kx_mla_attend_launch(&c, L.cache, seq_stride, m->qabs + (size_t)i0 * NB * c.heads * KVA, m->partial,
                                    m->o_lat + (size_t)i0 * NB * c.heads * c.kv_rank, np * NB, pos + i0 + np, st, C > 1 ? NB : 0, mla_kernel));
      }
    }
    if (C > 1 && B > 32 && c.kv_rank % 128 == 0) {  // a long prefill step: one grouped GEMM over the heads
      if (l == 0) {
        hipLaunchKernelGGL(head_groups_k, dim3(kx_cdiv(B * c.heads, 256)), dim3(256), 0, st, B, c.heads, m->head_work, m->head_pairs);
        KX_LAUNCH_CHECK();
      }
      KX_TRY(kx_grouped_gemm_launch(false, false, L.kvb + (size_t)c.qk_nope * c.kv_rank, nullptr, nullptr, nullptr, m->o_lat, m->att,
                                    KX_GG_BF16, m->head_work, m->head_pairs, 0, c.heads, c.v_head, c.kv_rank, 1,
                                    (size_t)(c.qk_nope + c.v_head) * c.kv_rank, 0, B, st));
      KxGemvArgs go = {};
      go.w0 = L.o; go.x = m->att; go.x_stride = VD; go.out = m->x; go.out_stride = H; go.rows = H; go.cols = VD; go.tokens = B;
      KX_TRY(dense(KX_EPI_RESID, go));                                                                  // :826-827
    } else {
      KxGemvArgs go = {};
      go.w0 = L.o; go.x = m->att; go.x_stride = VD; go.out = m->x; go.out_stride = H; go.rows = H; go.cols = VD; go.tokens = B;
      // One token: the merge of the attention partials, W_UV and o_proj with the residual add as one resident launch
      // where the shapes and the device allow it (kx_front.hip; same sums, same bits)
      // and, in front of a MoE layer, that layer's head too (post-attention norm, shared gate/up, router, routing)
      bool back = false;
      if (fuse && B == 1 && g.mla_po && (m->fusion & KX_FUSE_BACK)) {
        const uint32_t tag = m->back_tag % 65535u + 1u;
        KxMoeHeadArgs hd;
        const bool want_head = l >= c.first_dense && (m->fusion & KX_FUSE_MOE_HEAD);
        if (want_head) kx_moe_head_args(&c, &L.moe, m->moe_ws, m->n, L.post_ln, &hd);
        KX_TRY(kx_attn_back_launch(g, go, want_head ? &hd : nullptr, m->back_hand, tag, m->hand_err, &back, &moe_head_done, st));
        if (back) m->back_tag = tag;
      }
      if (!back) {
        KX_TRY(kx_gemv_launch(KX_EPI_BF16, g, st));
        KX_TRY(dense(KX_EPI_RESID, go));                                                                // :826-827
      }
    }
    if (l < c.first_dense) {                                                                            // bf16_mlp (:674-686)
      g = {};
      g.w0 = L.dgate; g.w1 = L.dup; g.x = m->n; g.x_stride = H; g.out = m->dmid; g.out_stride = c.dense_inter;
      g.rows = c.dense_inter; g.cols = H; g.tokens = B;
      if (fuse) { g.x = m->x; g.norm_w = L.post_ln; g.norm_eps = c.rms_eps; }
      else KX_TRY(kx_rmsnorm_launch(m->x, L.post_ln, m->n, B, H, H, H, c.rms_eps, st));                // :829
      KX_TRY(dense(KX_EPI_SWIGLU, g));
      g = {};
      g.w0 = L.ddown; g.x = m->dmid; g.x_stride = c.dense_inter; g.out = m->x; g.out_stride = H; g.rows = H;
      g.cols = c.dense_inter; g.tokens = B;
      KX_TRY(dense(KX_EPI_RESID, g));                                                                   // :684, :877
    } else {
      if (!fuse) KX_TRY(kx_rmsnorm_launch(m->x, L.post_ln, m->n, B, H, H, H, c.rms_eps, st));          // :829
      if (C > 1 && B > 32) {  // a prefill step of more than 32 tokens: the grouped GEMMs of the prefill layer
        KX_TRY(kx_moe_prefill_layer(&c, &L.moe, m->moe_ws, m->n, m->x, B, 0, st));
      } else {
        // From 12 tokens on the routed experts with several pairs run as grouped GEMMs: such an expert's weights are
        // streamed and dequantised once for all its tokens, where the GEMV kernels go over them once per token (from
        // L2, but at one fma per weight and token on the VALU); the experts with one pair keep the GEMV kernel, which
        // streams them faster than the GEMM kernel does at one token.  With 32 sequences that decode alike (70-100
        // distinct experts for 256 pairs, up to 23 pairs on one expert) the step goes from 24.5 to 18.1 ms; at 12
        // sequences the two forms are level (12.1 against 12.4 ms), at 8 the GEMV kernels win (9.8 against 10.9 ms).
        const uint32_t flags = ((m->fusion & KX_FUSE_MOE_TAIL) ? 0u : KX_MOE_SEPARATE_TAIL) | (moe_head_done ? KX_MOE_HEAD_DONE : 0u) |
                               ((m->fusion & KX_FUSE_ROUTED) ? KX_MOE_ROUTED_RESIDENT : 0u) | (B >= 5 && !(m->exact & KX_EXACT_SHARED) ? KX_MOE_SHARED_MATRIX_CORES : 0u) |
                               (B >= 12 && !(m->exact & KX_EXACT_ROUTED) ? KX_MOE_ROUTED_MATRIX_CORES : 0u);
        KX_TRY(kx_moe_layer_launch(&c, &L.moe, m->moe_ws, m->n, m->x, B, flags, fuse ? L.post_ln : nullptr, st, false));  // :835-877
      }
      if (m->route_logits) {  // the routing record: logits of the first rows and the number of distinct experts
        const int rows = B < c.max_batch ? B : c.max_batch;
        void *d_logits = nullptr;
        KX_TRY(kx_moe_workspace_views(m->moe_ws, &d_logits, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr));
        KX_HIP(hipMemcpyAsync(m->route_logits + (size_t)l * c.max_batch * c.experts, d_logits, (size_t)rows * c.experts * 4,
                              hipMemcpyDeviceToDevice, st));
        KX_HIP(hipMemcpyAsync(m->route_distinct + l, kx_moe_workspace_n_active(m->moe_ws), 4, hipMemcpyDeviceToDevice, st));
        if (m->route_history) {  // every token of the step: token i * NB + b is position pos + i of sequence b
          const size_t row = (size_t)c.experts * 4;
          KX_HIP(hipMemcpy2DAsync(m->route_history + (((size_t)l * c.max_context + pos) * c.max_batch) * c.experts, (size_t)c.max_batch * row,
                                  d_logits, (size_t)NB * row, (size_t)NB * row, (size_t)C, hipMemcpyDeviceToDevice, st));
        }
      }
    }
  }
  const uint16_t *x_last = m->x + (size_t)(C - 1) * NB * H;  // rows of the last position
  if (sample) {                                                                                          // :880-881
    KxGemvArgs g = {};
    g.w0 = m->lm_head; g.x = m->n; g.x_stride = H; g.out = m->logits; g.out_stride = c.vocab; g.rows = c.vocab; g.cols = H;
    g.tokens = NB;
    if (fuse) { g.x = m->x; g.norm_w = m->final_norm; g.norm_eps = c.rms_eps; }
    else KX_TRY(kx_rmsnorm_launch(x_last, m->final_norm, m->n, NB, H, H, H, c.rms_eps, st));
    KX_TRY(dense(KX_EPI_ARGMAX, g));
    KX_TRY(kx_argmax_launch(m->logits, NB, c.vocab, c.vocab, m->next, m->argmax_scratch, st));
  }
#undef KX_TRY
  m->sampled = sample;
  m->pos = pos + C;
  m->x_row0 = (C - 1) * NB;
  return KX_OK;
}

}  // namespace

extern "C" int kx_model_bytes(const kx_config *cfg, uint64_t *weights, uint64_t *kv_cache, uint64_t *scratch) {
  int rc = check_model_cfg(cfg);
  if (rc) return rc;
  Plan p;
  layout(cfg, p, nullptr);
  if (weights) *weights = p.weights;
  if (kv_cache) *kv_cache = p.cache;
  if (scratch) *scratch = p.scratch;
  return KX_OK;
}

// allocates the arena, lays the model out and creates its stream, events and MoE workspace; weights are not set
static int model_new(const kx_config *cfg, const char *who, kx_model **out) {
  KX_REQUIRE(out, "%s: null out pointer", who);
  *out = nullptr;
  int rc = check_model_cfg(cfg);
  if (rc) return rc;
  Plan p;
  layout(cfg, p, nullptr);
  size_t free_b = 0, total_b = 0;
  KX_HIP(hipMemGetInfo(&free_b, &total_b));
  KX_REQUIRE(p.total + ((size_t)1 << 30) <= free_b, "%s: the model needs %.1f GB of HBM, %.1f GB are free", who,
             p.total / 1e9, free_b / 1e9);
  kx_model *m = new kx_model();
  m->c = *cfg;
  hipError_t e = hipMalloc((void **)&m->arena, p.total);
  if (e != hipSuccess) {
    kx_set_error("%s: hipMalloc(%zu): %s", who, p.total, hipGetErrorString(e));
    delete m;
    return KX_ERR_HIP;
  }
  m->arena_bytes = p.total;
  Plan p2;
  layout(cfg, p2, m);
  rc = KX_OK;
  if (hipStreamCreate(&m->st) != hipSuccess) rc = KX_ERR_HIP;
  for (auto &ev : m->ev)
    if (!rc && hipEventCreate(&ev) != hipSuccess) rc = KX_ERR_HIP;
  if (!rc && cfg->first_dense < cfg->n_layers) rc = kx_moe_workspace_create(cfg, step_tokens(cfg), &m->moe_ws);
  if (!rc && m->moe_ws) kx_moe_workspace_set_err(m->moe_ws, m->hand_err);
  if (!rc && (hipMemsetAsync(m->head_count, 0, (size_t)cfg->heads * 4, m->st) != hipSuccess ||
              hipMemsetAsync(m->hand_err, 0, 4, m->st) != hipSuccess ||
              hipMemsetAsync(m->back_hand, 0, kx_back_hand_words(cfg->heads * cfg->v_head, cfg->hidden, cfg->experts) * 4, m->st) != hipSuccess ||
              hipMemsetAsync(m->front_hand, 0, kx_front_hand_words(cfg->q_rank, cfg->kv_rank + cfg->qk_rope, cfg->heads * (cfg->qk_nope + cfg->qk_rope)) * 4, m->st) != hipSuccess || hipStreamSynchronize(m->st) != hipSuccess))
    rc = KX_ERR_HIP;
  if (rc) {
    if (rc == KX_ERR_HIP && !kx_last_error()[0]) kx_set_error("%s: HIP resource creation failed", who);
    kx_model_destroy(m);
    return rc;
  }
  *out = m;
  return KX_OK;
}

extern "C" int kx_model_create(const kx_config *cfg, kx_model **out) {
  kx_model *m = nullptr;
  int rc = model_new(cfg, "kx_model_create", &m);
  if (rc) return rc;
  if ((rc = init_weights(m))) {
    kx_model_destroy(m);
    return rc;
  }
  *out = m;
  return KX_OK;
}

// where checkpoint tensor `n` lives in the arena
static char *need_dst(kx_model *m, const KxNeed &n) {
  const kx_config &c = m->c;
  const size_t H = c.hidden, I = c.moe_inter, e = n.expert < 0 ? 0 : (size_t)n.expert;
  if (n.layer < 0) return (char *)(n.slot == KXS_EMBED ? m->embed : n.slot == KXS_FINAL_NORM ? m->final_norm : m->lm_head);
  Layer &L = m->layers[n.layer];
  const kx_moe_weights &w = L.moe;
  switch (n.slot) {
    case KXS_INPUT_LN: return (char *)L.input_ln;
    case KXS_QA: return (char *)L.qkv_a;
    case KXS_KVA: return (char *)(L.qkv_a + (size_t)c.q_rank * H);  // kv_a rows follow the q_a rows: one GEMV reads both
    case KXS_QA_LN: return (char *)L.qa_ln;
    case KXS_QB: return (char *)L.qb;
    case KXS_KV_LN: return (char *)L.kv_ln;
    case KXS_KVB: return (char *)L.kvb;  // rows h*(nope+v)+d: d < nope is W_UK[h], the rest W_UV[h] (split_kv_k, :364-370)
    case KXS_O: return (char *)L.o;
    case KXS_POST_LN: return (char *)L.post_ln;
    case KXS_DENSE_GATE: return (char *)L.dgate;
    case KXS_DENSE_UP: return (char *)L.dup;
    case KXS_DENSE_DOWN: return (char *)L.ddown;
    case KXS_ROUTER: return (char *)w.d_router_gate;
    case KXS_ROUTER_BIAS: return (char *)w.d_router_bias;
    case KXS_GATE_P: return (char *)w.d_gate_packed + e * (I * H / 2);
    case KXS_GATE_S: return (char *)w.d_gate_scale + e * (I * H / 16);
    case KXS_UP_P: return (char *)w.d_up_packed + e * (I * H / 2);
    case KXS_UP_S: return (char *)w.d_up_scale + e * (I * H / 16);
    case KXS_DOWN_P: return (char *)w.d_down_packed + e * (H * I / 2);
    case KXS_DOWN_S: return (char *)w.d_down_scale + e * (H * I / 16);
    case KXS_SH_GATE: return (char *)w.d_shared_gate;
    case KXS_SH_UP: return (char *)w.d_shared_up;
    case KXS_SH_DOWN: return (char *)w.d_shared_down;
    default: return nullptr;
  }
}

extern "C" int kx_model_load(const kx_config *cfg, const char *index_path, kx_model **out) {
  KX_REQUIRE(out, "kx_model_load: null out pointer");
  *out = nullptr;
  KX_REQUIRE(cfg, "kx_model_load: null config");
  KxIndex ix;
  int rc = kx_index_parse(index_path, ix);
  if (rc) return rc;
  std::vector<KxNeed> needs;
  if ((rc = check_model_cfg(cfg)) || (rc = kx_index_contract(ix, cfg, needs))) return rc;
  kx_model *m = nullptr;
  if ((rc = model_new(cfg, "kx_model_load", &m))) return rc;
  std::vector<KxLoadItem> items;
  items.reserve(needs.size());
  for (const KxNeed &n : needs) {
    KxLoadItem it;
    it.t = n.t;
    it.dst = need_dst(m, n);
    it.widen = n.slot == KXS_ROUTER_BIAS;  // the router keeps the bias in f32; the checkpoint's bf16 widens exactly
    items.push_back(it);
  }
  rc = kx_load_run(items, &m->load_bytes, &m->load_seconds);
  if (!rc) rc = init_rope(m);
  if (rc) {
    kx_model_destroy(m);
    return rc;
  }
  *out = m;
  return KX_OK;
}

extern "C" int kx_model_load_info(kx_model *m, uint64_t *bytes, double *seconds) {
  KX_REQUIRE(m, "kx_model_load_info: null model");
  if (bytes) *bytes = m->load_bytes;
  if (seconds) *seconds = m->load_seconds;
  return KX_OK;
}

extern "C" int kx_model_destroy(kx_model *m) {
  if (!m) return KX_OK;
  if (m->st) (void)hipStreamSynchronize(m->st);
  if (m->moe_ws) kx_moe_workspace_destroy(m->moe_ws);
  for (auto &ev : m->ev)
    if (ev) (void)hipEventDestroy(ev);
  if (m->st) (void)hipStreamDestroy(m->st);
  if (m->arena) (void)hipFree(m->arena);
  if (m->route_logits) (void)hipFree(m->route_logits);
  if (m->route_distinct) (void)hipFree(m->route_distinct);
  if (m->route_history) (void)hipFree(m->route_history);
  delete m;
  return KX_OK;
}

static int check_ids(const kx_model *m, const uint32_t *ids, size_t n) {
  for (size_t i = 0; i < n; ++i)
    KX_REQUIRE(ids[i] < (uint32_t)m->c.vocab, "token id %u outside the vocabulary of %d", ids[i], m->c.vocab);  // :552, :652
  return KX_OK;
}

// Synchronises the model's stream and reports a wait inside a resident launch (kx_front.hip, the routed experts'
// launch of kx_i4.hip) that was given up: the steps since then computed with values that were not there yet.
static int check_front(kx_model *m) {
  int flag = 0;
  KX_HIP(hipMemcpyAsync(&flag, m->hand_err, 4, hipMemcpyDeviceToHost, m->st));
  KX_HIP(hipStreamSynchronize(m->st));
  if (flag) {
    kx_set_error("kx_model: a workgroup of a resident launch gave up waiting for values from the others (not all workgroups of the launch "
                 "were on the device at once); results since then are invalid -- switch the resident launches off with "
                 "kx_model_set_fusion(model, KX_FUSE_ABSORB | KX_FUSE_MOE_TAIL)");
    return KX_ERR_STATE;
  }
  return KX_OK;
}

extern "C" int kx_prefill(kx_model *m, const uint32_t *h_ids, int32_t batch, int32_t prompt_len) {
  KX_REQUIRE(m && h_ids, "kx_prefill: null argument");
  KX_REQUIRE(batch > 0 && batch <= m->c.max_batch, "kx_prefill: batch=%d outside [1, %d]", batch, m->c.max_batch);
  KX_REQUIRE(prompt_len > 0 && prompt_len <= m->c.max_context, "kx_prefill: prompt_len=%d outside [1, %d]", prompt_len, m->c.max_context);  // :555, :784
  int rc = check_ids(m, h_ids, (size_t)batch * prompt_len);
  if (rc) return rc;
  std::vector<uint32_t> pm((size_t)prompt_len * batch);  // position-major
  for (int b = 0; b < batch; ++b)
    for (int i = 0; i < prompt_len; ++i) pm[(size_t)i * batch + b] = h_ids[(size_t)b * prompt_len + i];
  KX_HIP(hipMemcpyAsync(m->ids, pm.data(), pm.size() * 4, hipMemcpyHostToDevice, m->st));
  KX_HIP(hipStreamSynchronize(m->st));  // pm goes out of scope
  m->batch = batch;
  m->pos = 0;
  // :886: one run() per prompt token, sampling on the last; with a prefill chunk set, up to that many positions per step
  int chunk = m->prefill_chunk < STEP_TOKENS / batch ? m->prefill_chunk : STEP_TOKENS / batch;
  if (chunk < 1 || m->exact == KX_EXACT_ALL) chunk = 1;  // a step of several positions is a tolerance path
  for (int i = 0; i < prompt_len; i += chunk) {
    const int n = prompt_len - i < chunk ? prompt_len - i : chunk;
    if ((rc = step(m, m->ids + (size_t)i * batch, i + n == prompt_len, n))) return rc;
  }
  return KX_OK;
}

extern "C" int kx_decode_step(kx_model *m, const uint32_t *h_ids) {
  KX_REQUIRE(m, "kx_decode_step: null model");
  KX_REQUIRE(m->batch > 0, "kx_decode_step: no prefill has run");
  KX_REQUIRE(m->pos < m->c.max_context, "kx_decode_step: the context of %d positions is full", m->c.max_context);  // :784
  const uint32_t *src = m->next;
  if (h_ids) {
    int rc = check_ids(m, h_ids, m->batch);
    if (rc) return rc;
    uint32_t *slot = m->ids + (size_t)m->pos * m->batch;
    KX_HIP(hipMemcpyAsync(slot, h_ids, (size_t)m->batch * 4, hipMemcpyHostToDevice, m->st));
    KX_HIP(hipStreamSynchronize(m->st));
    src = slot;
  } else {
    KX_REQUIRE(m->sampled, "kx_decode_step: no sampled ids to feed (pass h_ids)");
    // the sampler overwrites `next`; feed a copy
    uint32_t *slot = m->ids + (size_t)m->pos * m->batch;
    hipLaunchKernelGGL(copy_ids_k, dim3(kx_cdiv(m->batch, 64)), dim3(64), 0, m->st, m->next, slot, m->batch);
    KX_LAUNCH_CHECK();
    src = slot;
  }
  return step(m, src, true);
}

extern "C" int kx_greedy_sample(kx_model *m, uint32_t *h_out) {
  KX_REQUIRE(m && h_out, "kx_greedy_sample: null argument");
  KX_REQUIRE(m->sampled, "kx_greedy_sample: the last step did not sample");
  KX_HIP(hipMemcpyAsync(h_out, m->next, (size_t)m->batch * 4, hipMemcpyDeviceToHost, m->st));
  return check_front(m);
}

extern "C" int kx_generate(kx_model *m, const uint32_t *h_prompt, int32_t batch, int32_t prompt_len, int32_t n_tokens,
                           int ignore_eos, uint32_t *h_out, int32_t *h_counts) {
  KX_REQUIRE(m && h_prompt && h_out && h_counts, "kx_generate: null argument");
  KX_REQUIRE(n_tokens > 0, "kx_generate: n_tokens=%d must be positive", n_tokens);  // :542
  KX_REQUIRE((int64_t)prompt_len + n_tokens <= m->c.max_context, "requested sequence exceeds the context of %d positions", m->c.max_context);  // :784
  int rc;
  KX_HIP(hipEventRecord(m->ev[0], m->st));
  if ((rc = kx_prefill(m, h_prompt, batch, prompt_len))) return rc;
  KX_HIP(hipEventRecord(m->ev[1], m->st));
  const int cp = kx_cdiv(batch, 64);
  // Steps are enqueued without waiting for the host.  When the end-of-sequence id counts, the ids sampled so far are
  // read back every eighth step, and the loop ends once every sequence has sampled it (:887-888 stop there too):
  // at most eight steps are decoded for nothing.
  std::vector<uint32_t> hist((size_t)n_tokens * batch);
  std::vector<char> ended(batch, 0);
  int made = 0, seen = 0;  // history rows written on the device, and of those, rows the host has read
  auto read_back = [&]() -> int {
    if (seen == made) return KX_OK;
    KX_HIP(hipMemcpyAsync(hist.data() + (size_t)seen * batch, m->history + (size_t)seen * batch, (size_t)(made - seen) * batch * 4,
                          hipMemcpyDeviceToHost, m->st));
    KX_HIP(hipStreamSynchronize(m->st));
    for (; seen < made; ++seen)
      for (int b = 0; b < batch; ++b)
        if (hist[(size_t)seen * batch + b] == m->c.eos_id) ended[b] = 1;
    return KX_OK;
  };
  for (int i = 0; i < n_tokens; ++i) {  // :887-890
    hipLaunchKernelGGL(copy_ids_k, dim3(cp), dim3(64), 0, m->st, m->next, m->history + (size_t)i * batch, batch);
    KX_LAUNCH_CHECK();
    made = i + 1;
    if (!ignore_eos && (i & 7) == 7) {
      if ((rc = read_back())) return rc;
      bool all = true;
      for (int b = 0; b < batch; ++b) all = all && ended[b];
      if (all) break;
    }
    if (i + 1 < n_tokens && (rc = step(m, m->history + (size_t)i * batch, true))) return rc;
  }
  KX_HIP(hipEventRecord(m->ev[2], m->st));
  if ((rc = read_back())) return rc;
  if ((rc = check_front(m))) return rc;
  KX_HIP(hipEventElapsedTime(&m->ms_prefill, m->ev[0], m->ev[1]));
  KX_HIP(hipEventElapsedTime(&m->ms_decode, m->ev[1], m->ev[2]));
  m->steps_decoded = made;
  for (int b = 0; b < batch; ++b) {  // generation stops before the end-of-sequence id is emitted (:887-888)
    int n = 0;
    for (int i = 0; i < made; ++i) {
      const uint32_t id = hist[(size_t)i * batch + b];
      if (!ignore_eos && id == m->c.eos_id) break;
      h_out[(size_t)b * n_tokens + n++] = id;
    }
    h_counts[b] = n;
  }
  return KX_OK;
}

extern "C" int kx_model_set_prefill_chunk(kx_model *m, int32_t positions) {
  KX_REQUIRE(m, "kx_model_set_prefill_chunk: null model");
  KX_REQUIRE(positions >= 1 && positions <= STEP_TOKENS, "kx_model_set_prefill_chunk: positions=%d outside [1, %d]", positions, STEP_TOKENS);
  m->prefill_chunk = positions;
  return KX_OK;
}

extern "C" int kx_model_set_exact(kx_model *m, uint32_t mask) {
  KX_REQUIRE(m, "kx_model_set_exact: null model");
  KX_REQUIRE(!(mask & ~(uint32_t)KX_EXACT_ALL), "kx_model_set_exact: unknown bits in mask 0x%x", mask);
  m->exact = mask;
  return KX_OK;
}

extern "C" int kx_model_rewind(kx_model *m, int32_t positions) {
  KX_REQUIRE(m, "kx_model_rewind: null model");
  KX_REQUIRE(m->batch > 0, "kx_model_rewind: no prefill has run");
  KX_REQUIRE(positions >= 0 && positions <= m->pos, "kx_model_rewind: positions=%d outside [0, %d]", positions, m->pos);
  m->pos -= positions;
  if (positions) m->sampled = false;  // the sampled ids belonged to the last position
  return KX_OK;
}

extern "C" int kx_model_debug_fail_waits(kx_model *m) {
  KX_REQUIRE(m, "kx_model_debug_fail_waits: null model");
  const int one = 1;
  KX_HIP(hipMemcpyAsync(m->hand_err, &one, 4, hipMemcpyHostToDevice, m->st));
  KX_HIP(hipStreamSynchronize(m->st));
  return KX_OK;
}

extern "C" int kx_model_set_attention_kernel(kx_model *m, int32_t kernel) {
  KX_REQUIRE(m, "kx_model_set_attention_kernel: null model");
  KX_REQUIRE(kernel >= KX_MLA_AUTO && kernel <= KX_MLA_MATRIX_CORES, "kx_model_set_attention_kernel: kernel=%d outside [0, 2]", kernel);
  KX_REQUIRE(kernel != KX_MLA_MATRIX_CORES || m->c.heads == 64, "kx_model_set_attention_kernel: the matrix-core kernel is built for 64 heads (model: %d)", m->c.heads);
  m->mla_kernel = kernel;
  return KX_OK;
}
extern "C" int kx_model_set_routing_record(kx_model *m, int on) {
  KX_REQUIRE(m, "kx_model_set_routing_record: null model");
  KX_REQUIRE(m->c.first_dense < m->c.n_layers, "kx_model_set_routing_record: the model has no MoE layer");
  KX_HIP(hipStreamSynchronize(m->st));
  KX_REQUIRE(on >= 0 && on <= 2, "kx_model_set_routing_record: level %d outside [0, 2]", on);
  if (on < 2 && m->route_history) {
    (void)hipFree(m->route_history);
    m->route_history = nullptr;
  }
  if (!on) {
    if (m->route_logits) (void)hipFree(m->route_logits);
    if (m->route_distinct) (void)hipFree(m->route_distinct);
    m->route_logits = nullptr; m->route_distinct = nullptr;
    return KX_OK;
  }
  if (on == 2 && !m->route_history) {
    const size_t bytes = (size_t)m->c.n_layers * m->c.max_context * m->c.max_batch * m->c.experts * 4;
    KX_HIP(hipMalloc((void **)&m->route_history, bytes));
    KX_HIP(hipMemset(m->route_history, 0, bytes));
  }
  if (m->route_logits) return KX_OK;
  const size_t nl = (size_t)m->c.n_layers;
  float *lg = nullptr;
  int *di = nullptr;
  KX_HIP(hipMalloc((void **)&lg, nl * m->c.max_batch * m->c.experts * 4));
  if (hipMalloc((void **)&di, nl * 4) != hipSuccess || hipMemset(di, 0, nl * 4) != hipSuccess ||
      hipMemset(lg, 0, nl * m->c.max_batch * m->c.experts * 4) != hipSuccess) {
    (void)hipFree(lg);
    if (di) (void)hipFree(di);
    kx_set_error("kx_model_set_routing_record: no memory for the record");
    return KX_ERR_HIP;
  }
  m->route_logits = lg; m->route_distinct = di;
  return KX_OK;
}
extern "C" int kx_model_routing(kx_model *m, int32_t layer, float *h_logits, int32_t *h_distinct) {
  KX_REQUIRE(m && m->route_logits, "kx_model_routing: null model, or kx_model_set_routing_record was not switched on");
  KX_REQUIRE(layer >= m->c.first_dense && layer < m->c.n_layers, "kx_model_routing: layer %d is not a MoE layer of this model", layer);
  KX_REQUIRE(m->batch > 0, "kx_model_routing: no step has run");
  if (h_logits)
    KX_HIP(hipMemcpyAsync(h_logits, m->route_logits + (size_t)layer * m->c.max_batch * m->c.experts, (size_t)m->batch * m->c.experts * 4,
                          hipMemcpyDeviceToHost, m->st));
  if (h_distinct) KX_HIP(hipMemcpyAsync(h_distinct, m->route_distinct + layer, 4, hipMemcpyDeviceToHost, m->st));
  KX_HIP(hipStreamSynchronize(m->st));
  return KX_OK;
}
extern "C" int kx_model_routing_history(kx_model *m, int32_t layer, int32_t pos0, int32_t n, float *h_logits) {
  KX_REQUIRE(m && h_logits && m->route_history, "kx_model_routing_history: null argument, or kx_model_set_routing_record is not at level 2");
  KX_REQUIRE(layer >= m->c.first_dense && layer < m->c.n_layers, "kx_model_routing_history: layer %d is not a MoE layer of this model", layer);
  KX_REQUIRE(pos0 >= 0 && n >= 0 && pos0 + n <= m->c.max_context, "kx_model_routing_history: positions [%d, %d) outside the context of %d", pos0, pos0 + n, m->c.max_context);
  KX_HIP(hipMemcpyAsync(h_logits, m->route_history + (((size_t)layer * m->c.max_context + pos0) * m->c.max_batch) * m->c.experts,
                        (size_t)n * m->c.max_batch * m->c.experts * 4, hipMemcpyDeviceToHost, m->st));
  KX_HIP(hipStreamSynchronize(m->st));
  return KX_OK;
}
extern "C" int kx_model_set_fusion(kx_model *m, uint32_t mask) {
  KX_REQUIRE(m, "kx_model_set_fusion: null model");
  KX_REQUIRE(!(mask & ~(uint32_t)KX_FUSE_ALL), "kx_model_set_fusion: unknown bits in mask 0x%x", mask);
  m->fusion = mask;
  return KX_OK;
}

extern "C" int kx_model_steps_decoded(kx_model *m, int32_t *steps) {
  KX_REQUIRE(m && steps, "kx_model_steps_decoded: null argument");
  *steps = m->steps_decoded;
  return KX_OK;
}

extern "C" int kx_model_timing(kx_model *m, float *ms2) {
  KX_REQUIRE(m && ms2, "kx_model_timing: null argument");
  ms2[0] = m->ms_prefill;
  ms2[1] = m->ms_decode;
  return KX_OK;
}

extern "C" int kx_model_hidden(kx_model *m, uint16_t *h_out) {
  KX_REQUIRE(m && h_out && m->batch > 0, "kx_model_hidden: null argument or no step has run");
  KX_HIP(hipMemcpyAsync(h_out, m->x + (size_t)m->x_row0 * m->c.hidden, (size_t)m->batch * m->c.hidden * 2, hipMemcpyDeviceToHost, m->st));
  KX_HIP(hipStreamSynchronize(m->st));
  return KX_OK;
}
extern "C" int kx_model_logits(kx_model *m, float *h_out) {
  KX_REQUIRE(m && h_out && m->sampled, "kx_model_logits: null argument or the last step did not sample");
  KX_HIP(hipMemcpyAsync(h_out, m->logits, (size_t)m->batch * m->c.vocab * 4, hipMemcpyDeviceToHost, m->st));
  KX_HIP(hipStreamSynchronize(m->st));
  return KX_OK;
}
extern "C" int kx_model_latent(kx_model *m, int32_t layer, int32_t seq_index, int32_t pos0, int32_t n, uint16_t *h_out) {
  KX_REQUIRE(m && h_out, "kx_model_latent: null argument");
  KX_REQUIRE(layer >= 0 && layer < m->c.n_layers && seq_index >= 0 && seq_index < m->c.max_batch && pos0 >= 0 && n >= 0 &&
                 pos0 + n <= m->c.max_context, "kx_model_latent: index out of range");
  const size_t KVA = m->c.kv_rank + m->c.qk_rope;
  KX_HIP(hipMemcpyAsync(h_out, m->layers[layer].cache + ((size_t)seq_index * m->c.max_context + pos0) * KVA, (size_t)n * KVA * 2,
                        hipMemcpyDeviceToHost, m->st));
  KX_HIP(hipStreamSynchronize(m->st));
  return KX_OK;
}
extern "C" int kx_model_stream(kx_model *m, void **stream) {
  KX_REQUIRE(m && stream, "kx_model_stream: null argument");
  *stream = (void *)m->st;
  return KX_OK;
}
