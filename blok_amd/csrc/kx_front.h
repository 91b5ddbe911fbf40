// kx_front.h -- launch interface of the resident launches around the attention of one token (kx_front.hip).
#pragma once
#include <hip/hip_runtime.h>
#include "kx_attn_parts.h"
#include "kx_dense.h"

// words of the `hand` array for a model: the tagged q_a, kv_a and q values of one token
inline size_t kx_front_hand_words(int q_rank, int kva, int q_rows) { return (size_t)q_rank + kva + q_rows; }
int kx_attn_front_launch(const KxGemvArgs &g_qkv, const KxGemvArgs &g_qb, const QAbsArgs &q, uint32_t *hand, uint32_t tag, int *err,
                         bool *done, hipStream_t st);

// The head of a MoE layer for one token, as the back launch can carry it along: what the router + shared gate/up
// launch of kx_moe.hip reads and writes (kx_moe_head_args fills it from a layer's weights and workspace).
struct KxMoeHeadArgs {
  const uint16_t *post_ln;         // post-attention RMSNorm weights [hidden]
  const uint16_t *w_gate, *w_up;   // the shared expert's gate and up matrices, bf16 [shared_inter, hidden]
  const uint16_t *w_router;        // bf16 [experts, hidden]
  const float *bias;               // router bias [experts]
  uint16_t *n_out;                 // the normed row [hidden], read by the routed experts' launch
  uint16_t *smid;                  // bf(silu(gate) * up) of the shared expert [shared_inter]
  float *logits;                   // [experts]
  uint16_t *ids;                   // the routing, as kxr::route_block leaves it
  float *weights;
  int *counts, *offsets, *pairs;
  int4 *work;
  int *n_active;
  int shared_inter, experts, topk;
  float routed_scale, eps;
};
struct kx_moe_workspace;
// fills `out` for one token of a layer: weights w, buffers of ws, normed row to d_n (kx_moe.hip)
void kx_moe_head_args(const kx_config *c, const kx_moe_weights *w, kx_moe_workspace *ws, void *d_n, const uint16_t *norm_w, KxMoeHeadArgs *out);
// words of the back launch's `hand` array: the attention output, the residual row, two per router logit
inline size_t kx_back_hand_words(int vd, int hidden, int experts) { return (size_t)vd + hidden + 2 * (size_t)experts; }
// head: nullptr, or the MoE head to run behind o_proj; *head_done says whether it was taken along
int kx_attn_back_launch(const KxGemvArgs &g_uv, const KxGemvArgs &g_o, const KxMoeHeadArgs *head, uint32_t *hand, uint32_t tag, int *err,
                        bool *done, bool *head_done, hipStream_t st);
