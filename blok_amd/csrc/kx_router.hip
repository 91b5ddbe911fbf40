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

namespace {

constexpr int MAX_EPL = 16;  // experts per lane: up to 1024 experts

__global__ void __launch_bounds__(64) router_topk_k(const float *__restrict__ logits, const float *__restrict__ bias,
                                                    uint16_t *__restrict__ ids, float *__restrict__ weights, int E,
                                                    int topk, float routed_scale) {
  const int tok = blockIdx.x, lane = threadIdx.x;
  const float *lg = logits + (size_t)tok * E;
  float sc[MAX_EPL], sel[MAX_EPL];
  const float NEG_INF = -__builtin_inff();
#pragma unroll
  for (int j = 0; j < MAX_EPL; ++j) {
    int e = lane + 64 * j;
    if (e < E) {
      sc[j] = kx_sigmoidf(lg[e]);
      sel[j] = sc[j] + bias[e];
    } else {
      sc[j] = 0.0f;
      sel[j] = NEG_INF;
    }
  }
  float sum = 0.0f;
  float my_w = 0.0f;  // lane k keeps the k-th winner's score
  for (int k = 0; k < topk; ++k) {
    float best = NEG_INF;
    int bi = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < MAX_EPL; ++j)
      if (sel[j] > best) { best = sel[j]; bi = lane + 64 * j; }
    for (int m = 32; m; m >>= 1) {
      float ov = __shfl_xor(best, m);
      int oi = __shfl_xor(bi, m);
      if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if (bi == 0x7fffffff) bi = 0;  // every candidate was -inf: the reference keeps id 0
    float s_win = 0.0f;
#pragma unroll
    for (int j = 0; j < MAX_EPL; ++j)
      if (bi == lane + 64 * j) { s_win = sc[j]; sel[j] = NEG_INF; }
    s_win = __shfl(s_win, bi & 63);
    sum += s_win;
    if (lane == k) my_w = s_win;
    if (lane == 0) ids[(size_t)tok * topk + k] = (uint16_t)bi;
  }
  if (lane < topk) weights[(size_t)tok * topk + lane] = my_w / (sum + 1.0e-20f) * routed_scale;
}

__global__ void __launch_bounds__(1024) bucket_k(const uint16_t *__restrict__ ids, int n_pairs, int E,
                                                 int *__restrict__ counts, int *__restrict__ offsets,
                                                 int *__restrict__ pairs, int *__restrict__ active,
                                                 int *__restrict__ n_active) {
  __shared__ int s_cnt[1024];
  __shared__ int s_off[1025];
  const int e = threadIdx.x;
  int cnt = 0;
  if (e < E)
    for (int p = 0; p < n_pairs; ++p) cnt += (ids[p] == e) ? 1 : 0;
  s_cnt[e] = cnt;
  __syncthreads();
  if (e == 0) {
    int run = 0, na = 0;
    for (int i = 0; i < E; ++i) {
      s_off[i] = run;
      if (s_cnt[i] > 0) active[na++] = i;
      run += s_cnt[i];
    }
    s_off[E] = run;
    offsets[E] = run;
    *n_active = na;
  }
  __syncthreads();
  if (e < E) {
    counts[e] = cnt;
    offsets[e] = s_off[e];
    int pos = s_off[e];
    for (int p = 0; p < n_pairs; ++p)
      if (ids[p] == e) pairs[pos++] = p;
  }
}

}  // namespace

int kx_router_topk_launch(const float *logits, const float *bias, uint16_t *ids, float *weights, int tokens,
                          int experts, int topk, float routed_scale, hipStream_t st) {
  KX_REQUIRE(tokens > 0, "kx_router_topk: tokens=%d must be positive", tokens);
  KX_REQUIRE(experts > 0 && experts <= 64 * MAX_EPL, "kx_router_topk: experts=%d outside [1, %d]", experts, 64 * MAX_EPL);
  KX_REQUIRE(topk > 0 && topk <= 64 && topk <= experts, "kx_router_topk: topk=%d outside [1, min(64, experts)]", topk);
  hipLaunchKernelGGL(router_topk_k, dim3(tokens), dim3(64), 0, st, logits, bias, ids, weights, experts, topk,
                     routed_scale);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

int kx_bucket_launch(const uint16_t *ids, int tokens, int experts, int topk, int *counts, int *offsets, int *pairs,
                     int *active, int *n_active, hipStream_t st) {
  KX_REQUIRE(tokens > 0 && topk > 0, "kx_bucket: tokens=%d topk=%d must be positive", tokens, topk);
  KX_REQUIRE(experts > 0 && experts <= 1024, "kx_bucket: experts=%d outside [1, 1024]", experts);
  int threads = kx_cdiv(experts, 64) * 64;
  hipLaunchKernelGGL(bucket_k, dim3(1), dim3(threads), 0, st, ids, tokens * topk, experts, counts, offsets, pairs,
                     active, n_active);
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
                         void *d_offsets, void *d_pairs, void *d_active, void *d_n_active, void *stream) {
  KX_REQUIRE(d_ids && d_counts && d_offsets && d_pairs && d_active && d_n_active, "kx_bucket: null pointer");
  return kx_bucket_launch((const uint16_t *)d_ids, tokens, experts, topk, (int *)d_counts, (int *)d_offsets,
                          (int *)d_pairs, (int *)d_active, (int *)d_n_active, kx_stream(stream));
}
