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
#include "kx_wave.h"

namespace {

using kxw::wave_max_f32;
using kxw::wave_min_i32;

// top-k of one token by one wave; lane owns experts lane, lane+64, ... (EPL of them)
template <int EPL>
__device__ __forceinline__ void topk_token(const float *__restrict__ lg, const float *__restrict__ bias,
                                           uint16_t *__restrict__ ids, float *__restrict__ weights, int E, int topk,
                                           float routed_scale, int lane) {
  float sc[EPL], sel[EPL];
  const float NEG_INF = -__builtin_inff();
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    int e = lane + 64 * j;
    float x = e < E ? lg[e] : 0.0f, b = e < E ? bias[e] : 0.0f;
    sc[j] = kx_sigmoidf(x);
    sel[j] = e < E ? sc[j] + b : NEG_INF;
  }
  float sum = 0.0f;
  float my_w = 0.0f;  // lane k keeps the k-th winner's score
  for (int k = 0; k < topk; ++k) {
    float best = NEG_INF;
    int bi = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < EPL; ++j)
      if (sel[j] > best) { best = sel[j]; bi = lane + 64 * j; }
    const float m = wave_max_f32(best);
    int win = wave_min_i32(best == m ? bi : 0x7fffffff);
    if (win == 0x7fffffff) win = 0;  // every candidate was -inf: the reference keeps id 0 (:391-393)
    float s_win = 0.0f;
#pragma unroll
    for (int j = 0; j < EPL; ++j)
      if (win == lane + 64 * j) { s_win = sc[j]; sel[j] = NEG_INF; }
    s_win = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, s_win), win & 63));
    sum += s_win;
    if (lane == k) my_w = s_win;
    if (lane == 0) ids[k] = (uint16_t)win;
  }
  if (lane < topk) weights[lane] = my_w / (sum + 1.0e-20f) * routed_scale;
}

// one wave per token
template <int EPL>
__global__ void __launch_bounds__(64) router_topk_k(const float *__restrict__ logits, const float *__restrict__ bias,
                                                    uint16_t *__restrict__ ids, float *__restrict__ weights, int E,
                                                    int topk, float routed_scale) {
  const int tok = blockIdx.x;
  topk_token<EPL>(logits + (size_t)tok * E, bias, ids + (size_t)tok * topk, weights + (size_t)tok * topk, E, topk,
                  routed_scale, threadIdx.x);
}

// one workgroup, thread e owns expert e: count, exclusive scan, stable placement.
// The ids are staged in LDS (padded with 0xffff to a multiple of 8) and scanned 8 at a time.
__device__ __forceinline__ void bucket_block(const uint16_t *__restrict__ ids, int n_pairs, int E,
                                             int *__restrict__ counts, int *__restrict__ offsets,
                                             int *__restrict__ pairs, int4 *__restrict__ work,
                                             int *__restrict__ n_active, uint4 *s_ids4, int *s_cnt, int *s_act) {
  const int e = threadIdx.x, n = blockDim.x;
  const int n8 = (n_pairs + 7) >> 3;
  uint16_t *s_ids = (uint16_t *)s_ids4;
  for (int p = threadIdx.x; p < n8 * 8; p += n) s_ids[p] = p < n_pairs ? ids[p] : (uint16_t)0xffff;
  __syncthreads();
  const uint32_t me = (uint32_t)e, me2 = me | (me << 16);
  int cnt = 0;
  if (e < E)
    for (int q = 0; q < n8; ++q) {
      const uint4 u = s_ids4[q];
      const uint32_t w[4] = {u.x ^ me2, u.y ^ me2, u.z ^ me2, u.w ^ me2};
#pragma unroll
      for (int j = 0; j < 4; ++j) cnt += ((w[j] & 0xffffu) == 0) + ((w[j] >> 16) == 0);
    }
  s_cnt[e] = cnt;
  s_act[e] = cnt > 0 ? 1 : 0;
  __syncthreads();
  for (int d = 1; d < n; d <<= 1) {  // inclusive Hillis-Steele scans of both arrays
    int a = e >= d ? s_cnt[e - d] : 0, b = e >= d ? s_act[e - d] : 0;
    __syncthreads();
    s_cnt[e] += a;
    s_act[e] += b;
    __syncthreads();
  }
  const int off = s_cnt[e] - cnt, slot = s_act[e] - (cnt > 0 ? 1 : 0), total_active = s_act[n - 1];
  if (e < E) {
    counts[e] = cnt;
    offsets[e] = off;
    int pos = off, first = 0;
    if (cnt > 0)
      for (int q = 0; q < n8 && pos < off + cnt; ++q) {
        const uint4 u = s_ids4[q];
        const uint32_t w[4] = {u.x ^ me2, u.y ^ me2, u.z ^ me2, u.w ^ me2};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint32_t h = (j & 1) ? (w[j >> 1] >> 16) : (w[j >> 1] & 0xffffu);
          if (h == 0) {
            if (pos == off) first = q * 8 + j;
            pairs[pos++] = q * 8 + j;
          }
        }
      }
    if (cnt > 0) work[slot] = make_int4(e, off, off + cnt, first);
    if (e >= total_active) work[e] = make_int4(-1, 0, 0, 0);
  }
  if (e == 0) {
    offsets[E] = s_cnt[n - 1];
    *n_active = total_active;
  }
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

// top-k of up to blockDim/64 tokens (one wave each), then the bucketing, in one workgroup
template <int EPL>
__global__ void __launch_bounds__(1024) topk_bucket_k(const float *__restrict__ logits, const float *__restrict__ bias,
                                                      uint16_t *__restrict__ ids, float *__restrict__ weights, int tokens,
                                                      int E, int topk, float routed_scale, int *__restrict__ counts,
                                                      int *__restrict__ offsets, int *__restrict__ pairs,
                                                      int4 *__restrict__ work, int *__restrict__ n_active) {
  extern __shared__ uint4 s_ids4[];
  __shared__ int s_cnt[1024];
  __shared__ int s_act[1024];
  const int wave = threadIdx.x >> 6;
  if (wave < tokens)
    topk_token<EPL>(logits + (size_t)wave * E, bias, ids + (size_t)wave * topk, weights + (size_t)wave * topk, E, topk,
                    routed_scale, threadIdx.x & 63);
  __threadfence_block();
  __syncthreads();  // the ids written above are read back by bucket_block
  bucket_block(ids, tokens * topk, E, counts, offsets, pairs, work, n_active, s_ids4, s_cnt, s_act);
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
