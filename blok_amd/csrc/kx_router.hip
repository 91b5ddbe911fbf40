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
                                                 int *__restrict__ n_active, int4 *__restrict__ pair_work) {
  extern __shared__ uint4 s_ids4[];  // ceil(n_pairs / 8) pieces
  __shared__ int s_cnt[1024];
  __shared__ int s_act[1024];
  bucket_block(ids, n_pairs, E, counts, offsets, pairs, work, n_active, s_ids4, s_cnt, s_act, false, pair_work);
}

// top-k of the tokens (one wave each, in turns), then the bucketing, in one workgroup
template <int EPL>
__global__ void __launch_bounds__(1024) topk_bucket_k(const float *__restrict__ logits, const float *__restrict__ bias,
                                                      uint16_t *__restrict__ ids, float *__restrict__ weights, int tokens,
                                                      int E, int topk, float routed_scale, int *__restrict__ counts,
                                                      int *__restrict__ offsets, int *__restrict__ pairs,
                                                      int4 *__restrict__ work, int *__restrict__ n_active,
                                                      int4 *__restrict__ pair_work) {
  extern __shared__ uint4 s_ids4[];
  __shared__ int s_cnt[1024];
  __shared__ int s_act[1024];
  kxr::route_block<EPL, false, true>(logits, bias, ids, weights, tokens, E, topk, routed_scale, counts, offsets, pairs, work, n_active,
                        s_ids4, s_cnt, s_act, pair_work);
}

// ---- bucketing of a prefill chunk: one workgroup per expert instead of one per launch ------------
// ids of segment `seg` (seg_len a multiple of 8) compared with expert e; calls f(pair index) for every match, in order
template <typename F>
__device__ __forceinline__ void for_matches(const uint16_t *__restrict__ ids, int n_pairs, int begin, int end, uint32_t e, F f) {
  for (int p0 = begin; p0 < end; p0 += 8) {
    uint16_t v[8];
    if (p0 + 8 <= n_pairs) {
      const uint4 u = *(const uint4 *)(ids + p0);
      const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (uint16_t)((j & 1) ? (w[j >> 1] >> 16) : (w[j >> 1] & 0xffffu));
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = p0 + j < n_pairs ? ids[p0 + j] : (uint16_t)0xffff;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (v[j] == e) f(p0 + j);
  }
}

__device__ __forceinline__ int block_sum_256(int v, int *s_red) {  // sum over the 256 threads, returned to all
  for (int m = 32; m; m >>= 1) v += __shfl_xor(v, m);
  if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = v;
  __syncthreads();
  const int t = s_red[0] + s_red[1] + s_red[2] + s_red[3];
  __syncthreads();
  return t;
}

// grid (E), 256 threads: counts[e]
__global__ void __launch_bounds__(256) bucket_count_k(const uint16_t *__restrict__ ids, int n_pairs, int *__restrict__ counts) {
  __shared__ int s_red[4];
  const int seg = (((n_pairs + 255) >> 8) + 7) & ~7;
  int cnt = 0;
  for_matches(ids, n_pairs, threadIdx.x * seg, min(n_pairs, (threadIdx.x + 1) * seg), blockIdx.x, [&](int) { ++cnt; });
  cnt = block_sum_256(cnt, s_red);
  if (threadIdx.x == 0) counts[blockIdx.x] = cnt;
}

// one workgroup of at least E threads: offsets, the list of experts with work, n_active
__global__ void __launch_bounds__(1024) bucket_scan_k(const int *__restrict__ counts, int E, int *__restrict__ offsets,
                                                      int4 *__restrict__ work, int *__restrict__ n_active) {
  __shared__ int s_cnt[1024];
  __shared__ int s_act[1024];
  const int e = threadIdx.x, n = blockDim.x;
  const int cnt = e < E ? counts[e] : 0;
  s_cnt[e] = cnt;
  s_act[e] = cnt > 0 ? 1 : 0;
  __syncthreads();
  for (int d = 1; d < n; d <<= 1) {
    int a = e >= d ? s_cnt[e - d] : 0, b = e >= d ? s_act[e - d] : 0;
    __syncthreads();
    s_cnt[e] += a;
    s_act[e] += b;
    __syncthreads();
  }
  const int off = s_cnt[e] - cnt, slot = s_act[e] - (cnt > 0 ? 1 : 0), total_active = s_act[n - 1];
  if (e < E) {
    offsets[e] = off;
    if (cnt > 0) work[slot] = make_int4(e, off, off + cnt, 0);  // the first pair is filled in by bucket_place_k
    if (e >= total_active) work[e] = make_int4(-1, 0, 0, 0);
  }
  if (e == 0) {
    offsets[E] = s_cnt[n - 1];
    *n_active = total_active;
  }
}

// grid (E), 256 threads: the pairs of expert e in ascending order at pairs[offsets[e] ..]
__global__ void __launch_bounds__(256) bucket_place_k(const uint16_t *__restrict__ ids, int n_pairs, const int *__restrict__ counts,
                                                      const int *__restrict__ offsets, const int *__restrict__ n_active,
                                                      int *__restrict__ pairs, int4 *__restrict__ work) {
  __shared__ int s_scan[256];
  const int e = blockIdx.x, t = threadIdx.x;
  if (counts[e] == 0) return;
  const int off = offsets[e];
  const int seg = (((n_pairs + 255) >> 8) + 7) & ~7;
  const int begin = t * seg, end = min(n_pairs, (t + 1) * seg);
  int cnt = 0;
  for_matches(ids, n_pairs, begin, end, e, [&](int) { ++cnt; });
  s_scan[t] = cnt;
  __syncthreads();
  for (int d = 1; d < 256; d <<= 1) {
    const int a = t >= d ? s_scan[t - d] : 0;
    __syncthreads();
    s_scan[t] += a;
    __syncthreads();
  }
  int pos = off + s_scan[t] - cnt;
  const bool has_first = cnt > 0 && pos == off;
  int first = 0;
  for_matches(ids, n_pairs, begin, end, e, [&](int p) {
    if (pos == off) first = p;
    pairs[pos++] = p;
  });
  if (has_first) {  // the record of expert e: the list is sorted by expert id
    int lo = 0, hi = *n_active - 1;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (work[mid].x < e) lo = mid + 1;
      else hi = mid;
    }
    work[lo].w = first;
  }
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
                     int4 *work, int *n_active, hipStream_t st, int4 *pair_work) {
  KX_REQUIRE(tokens > 0 && topk > 0, "kx_bucket: tokens=%d topk=%d must be positive", tokens, topk);
  KX_REQUIRE(experts > 0 && experts <= 1024, "kx_bucket: experts=%d outside [1, 1024]", experts);
  int threads = kx_cdiv(experts, 64) * 64;
  const long n_pairs = (long)tokens * topk;
  KX_REQUIRE(n_pairs < (1L << 30), "kx_bucket: %ld pairs", n_pairs);
  KX_REQUIRE(!pair_work || n_pairs <= 1024, "kx_bucket: the per-pair work list is written for up to 1024 pairs (got %ld)", n_pairs);
  if (n_pairs > 1024) {  // a chunk: one workgroup per expert counts, one scans, one per expert places
    hipLaunchKernelGGL(bucket_count_k, dim3(experts), dim3(256), 0, st, ids, (int)n_pairs, counts);
    KX_LAUNCH_CHECK();
    hipLaunchKernelGGL(bucket_scan_k, dim3(1), dim3(threads), 0, st, counts, experts, offsets, work, n_active);
    KX_LAUNCH_CHECK();
    hipLaunchKernelGGL(bucket_place_k, dim3(experts), dim3(256), 0, st, ids, (int)n_pairs, counts, offsets, n_active, pairs, work);
    KX_LAUNCH_CHECK();
    return KX_OK;
  }
  const size_t lds = (size_t)kx_cdiv((int)n_pairs, 8) * 16;
  hipLaunchKernelGGL(bucket_k, dim3(1), dim3(threads), lds, st, ids, (int)n_pairs, experts, counts, offsets, pairs,
                     work, n_active, pair_work);
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
                          (int *)d_pairs, (int4 *)d_work, (int *)d_n_active, kx_stream(stream), nullptr);
}

// top-k and bucketing; one launch up to 32 tokens (one workgroup of up to 16 waves, each taking tokens in turn), two otherwise
int kx_route_launch(const float *logits, const float *bias, uint16_t *ids, float *weights, int tokens, int experts,
                    int topk, float routed_scale, int *counts, int *offsets, int *pairs, int4 *work, int *n_active,
                    hipStream_t st, int4 *pair_work) {
  if (tokens > 32 || experts > 1024 || (long)tokens * topk > 1024) {
    int rc = kx_router_topk_launch(logits, bias, ids, weights, tokens, experts, topk, routed_scale, st);
    if (rc) return rc;
    return kx_bucket_launch(ids, tokens, experts, topk, counts, offsets, pairs, work, n_active, st, pair_work);
  }
  KX_REQUIRE(tokens > 0 && experts > 0 && topk > 0 && topk <= 64 && topk <= experts, "kx_route: tokens=%d experts=%d topk=%d", tokens, experts, topk);
  int threads = kx_cdiv(experts, 64) * 64;
  if (threads < tokens * 64) threads = tokens * 64 < 1024 ? tokens * 64 : 1024;
  const size_t lds = (size_t)kx_cdiv(tokens * topk, 8) * 16;
  const int epl = kx_cdiv(experts, 64);
#define KX_TB(N) hipLaunchKernelGGL(topk_bucket_k<N>, dim3(1), dim3(threads), lds, st, logits, bias, ids, weights, tokens, experts, topk, routed_scale, counts, offsets, pairs, work, n_active, pair_work)
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
