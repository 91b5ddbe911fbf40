// kx_router.hip -- sigmoid / noaux-bias top-k router and token -> expert bucketing.
//
// Reference: sigmoid_k (src/kimi_exec.cu:377-380), add_bf16_k (:372-375),
// router_topk_k (:382-397): scores = sigmoid(logits); select = scores + bias;
// topk times: argmax of select with a strict '>' scan from index 0, so the
// lowest index wins ties; weights are the un-biased scores of the winners,
// divided by (their sum + 1e-20) and multiplied by the routed scaling factor.
// The reference does all of this on one thread and copies the ids to the host
// (:843-844); here one wave handles a token and the ids stay on the device.
//
// Bucketing has no counterpart in the reference (batch 1: the host loop at
// :845 is the bucket).  Canonical order: pairs (token*topk + slot) sorted by
// (expert, token, slot).
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_math.h"
#include "kx_route.h"
#include "kx_wave.h"

namespace {

using kxr::bucket_block;
using kxr::topk_token;

// one wave per token
template <int EPL>
__global__ void __launch_bounds__(64) router_topk_k(const float *__restrict__ logits, const float *__restrict__ bias,
                                                    uint16_t *__restrict__ ids, float *__restrict__ weights, int E,
                                                    int topk, float routed_scale) {
  const int tok = blockIdx.x;
  topk_token<EPL>(logits + (size_t)tok * E, bias, ids + (size_t)tok * topk, weights + (size_t)tok * topk, E, topk,
                  routed_scale, threadIdx.x);
}

__global__ void __launch_bounds__(1024) bucket_k(const uint16_t *__restrict__ ids, int n_pairs, int E,
                                                 int *__restrict__ counts, int *__restrict__ offsets,
                                                 int *__restrict__ pairs, int4 *__restrict__ work,
                                                 int *__restrict__ n_active) {
  extern __shared__ uint4 s_ids4[];  // ceil(n_pairs / 8) pieces
  __shared__ int s_cnt[1024];
  __shared__ int s_act[1024];
  bucket_block(ids, n_pairs, E, counts, offsets, pairs, work, n_active, s_ids4, s_cnt, s_act);
}

// top-k of the tokens (one wave each, in turns), then the bucketing, in one workgroup
template <int EPL>
__global__ void __launch_bounds__(1024) topk_bucket_k(const float *__restrict__ logits, const float *__restrict__ bias,
                                                      uint16_t *__restrict__ ids, float *__restrict__ weights, int tokens,
                                                      int E, int topk, float routed_scale, int *__restrict__ counts,
                                                      int *__restrict__ offsets, int *__restrict__ pairs,
                                                      int4 *__restrict__ work, int *__restrict__ n_active) {
  extern __shared__ uint4 s_ids4[];
  __shared__ int s_cnt[1024];
  __shared__ int s_act[1024];
  kxr::route_block<EPL>(logits, bias, ids, weights, tokens, E, topk, routed_scale, counts, offsets, pairs, work, n_active,
                        s_ids4, s_cnt, s_act);
}

}  // namespace

int kx_router_topk_launch(const float *logits, const float *bias, uint16_t *ids, float *weights, int tokens,
                          int experts, int topk, float routed_scale, hipStream_t st) {
  KX_REQUIRE(tokens > 0, "kx_router_topk: tokens=%d must be positive", tokens);
  KX_REQUIRE(experts > 0 && experts <= 1024, "kx_router_topk: experts=%d outside [1, %d]", experts, 1024);
  KX_REQUIRE(topk > 0 && topk <= 64 && topk <= experts, "kx_router_topk: topk=%d outside [1, min(64, experts)]", topk);
  const int epl = kx_cdiv(experts, 64);
#define KX_RT(N) hipLaunchKernelGGL(router_topk_k<N>, dim3(tokens), dim3(64), 0, st, logits, bias, ids, weights, experts, topk, routed_scale)
  if (epl <= 1) KX_RT(1);
  else if (epl <= 2) KX_RT(2);
  else if (epl <= 4) KX_RT(4);
  else if (epl <= 6) KX_RT(6);
  else if (epl <= 8) KX_RT(8);
  else KX_RT(16);
#undef KX_RT
  KX_LAUNCH_CHECK();
  return KX_OK;
}

int kx_bucket_launch(const uint16_t *ids, int tokens, int experts, int topk, int *counts, int *offsets, int *pairs,
                     int4 *work, int *n_active, hipStream_t st) {
  KX_REQUIRE(tokens > 0 && topk > 0, "kx_bucket: tokens=%d topk=%d must be positive", tokens, topk);
  KX_REQUIRE(experts > 0 && experts <= 1024, "kx_bucket: experts=%d outside [1, 1024]", experts);
  int threads = kx_cdiv(experts, 64) * 64;
  const size_t lds = (size_t)kx_cdiv(tokens * topk, 8) * 16;
  KX_REQUIRE(lds <= 48 * 1024, "kx_bucket: %d pairs exceed the %d the bucketing kernel stages", tokens * topk, 24576);
  hipLaunchKernelGGL(bucket_k, dim3(1), dim3(threads), lds, st, ids, tokens * topk, experts, counts, offsets, pairs,
                     work, n_active);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

extern "C" int kx_router_topk(const void *d_logits, const void *d_bias, void *d_ids, void *d_weights, int32_t tokens,
                              int32_t experts, int32_t topk, float routed_scale, void *stream) {
  KX_REQUIRE(d_logits && d_bias && d_ids && d_weights, "kx_router_topk: null pointer");
  return kx_router_topk_launch((const float *)d_logits, (const float *)d_bias, (uint16_t *)d_ids, (float *)d_weights,
                               tokens, experts, topk, routed_scale, kx_stream(stream));
}

extern "C" int kx_bucket(const void *d_ids, int32_t tokens, int32_t experts, int32_t topk, void *d_counts,
                         void *d_offsets, void *d_pairs, void *d_work, void *d_n_active, void *stream) {
  KX_REQUIRE(d_ids && d_counts && d_offsets && d_pairs && d_work && d_n_active, "kx_bucket: null pointer");
  return kx_bucket_launch((const uint16_t *)d_ids, tokens, experts, topk, (int *)d_counts, (int *)d_offsets,
                          (int *)d_pairs, (int4 *)d_work, (int *)d_n_active, kx_stream(stream));
}

// top-k and bucketing; one launch when the tokens fit one workgroup (16 waves), two otherwise
int kx_route_launch(const float *logits, const float *bias, uint16_t *ids, float *weights, int tokens, int experts,
                    int topk, float routed_scale, int *counts, int *offsets, int *pairs, int4 *work, int *n_active,
                    hipStream_t st) {
  if (tokens > 16 || experts > 1024) {
    int rc = kx_router_topk_launch(logits, bias, ids, weights, tokens, experts, topk, routed_scale, st);
    if (rc) return rc;
    return kx_bucket_launch(ids, tokens, experts, topk, counts, offsets, pairs, work, n_active, st);
  }
  KX_REQUIRE(tokens > 0 && experts > 0 && topk > 0 && topk <= 64 && topk <= experts, "kx_route: tokens=%d experts=%d topk=%d", tokens, experts, topk);
  int threads = kx_cdiv(experts, 64) * 64;
  if (threads < tokens * 64) threads = tokens * 64;
  const size_t lds = (size_t)kx_cdiv(tokens * topk, 8) * 16;
  const int epl = kx_cdiv(experts, 64);
#define KX_TB(N) hipLaunchKernelGGL(topk_bucket_k<N>, dim3(1), dim3(threads), lds, st, logits, bias, ids, weights, tokens, experts, topk, routed_scale, counts, offsets, pairs, work, n_active)
  if (epl <= 1) KX_TB(1);
  else if (epl <= 2) KX_TB(2);
  else if (epl <= 4) KX_TB(4);
  else if (epl <= 6) KX_TB(6);
  else if (epl <= 8) KX_TB(8);
  else KX_TB(16);
#undef KX_TB
  KX_LAUNCH_CHECK();
  return KX_OK;
}
