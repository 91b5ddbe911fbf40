// kx_route.h -- device-side pieces of the router: top-k of one token by one wave, and
// the token -> expert bucketing by one workgroup.  Shared by the stand-alone router
// kernels and by the GEMV whose last workgroup routes the logits it has just produced.
#pragma once
#include "kx_arrive.h"
#include "kx_common.h"
#include "kx_math.h"
#include "kx_wave.h"

namespace kxr {

using kxw::wave_max_f32;
using kxw::wave_min_i32;

// top-k of one token by one wave; lane owns experts lane, lane+64, ... (EPL of them).  COHERENT: the logits were
// written by other workgroups of the launch; HAND_IDS: the ids are read by another workgroup of the launch
template <int EPL, bool COHERENT = false, bool HAND_IDS = false>
__device__ __forceinline__ void topk_token(const float *lg, const float *__restrict__ bias,
                                           uint16_t *__restrict__ ids, float *__restrict__ weights, int E, int topk,
                                           float routed_scale, int lane, uint16_t *s_ids = nullptr) {
  float sc[EPL], sel[EPL];
  const float NEG_INF = -__builtin_inff();
  // all logits and biases of the lane are requested before the first is used (lanes past E read expert E - 1 and
  // drop it): with the load inside the loop below, each of the EPL sigmoids waited for its own round trip
  float x[EPL], bs[EPL];
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int ec = min(lane + 64 * j, E - 1);
    x[j] = COHERENT ? kx_arrive_load(lg + ec) : lg[ec];
    bs[j] = bias[ec];
  }
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    sc[j] = kx_sigmoidf(x[j]);
    sel[j] = lane + 64 * j < E ? sc[j] + bs[j] : NEG_INF;
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
    if (lane == 0) {
      if (HAND_IDS) kx_arrive_store(ids + k, (uint16_t)win);
      else ids[k] = (uint16_t)win;
      if (s_ids) s_ids[k] = (uint16_t)win;
    }
  }
  if (lane < topk) weights[lane] = my_w / (sum + 1.0e-20f) * routed_scale;
}

// topk_token with the per-lane expert count chosen at run time (up to 512 experts)
template <bool COHERENT, bool HAND_IDS>
__device__ __forceinline__ void topk_token_any(const float *lg, const float *bias, uint16_t *ids, float *weights, int E,
                                               int topk, float routed_scale, int lane) {
  const int epl = (E + 63) >> 6;
#define KX_TK(N) topk_token<N, COHERENT, HAND_IDS>(lg, bias, ids, weights, E, topk, routed_scale, lane)
  if (epl <= 1) KX_TK(1);
  else if (epl <= 2) KX_TK(2);
  else if (epl <= 4) KX_TK(4);
  else if (epl <= 6) KX_TK(6);
  else KX_TK(8);
#undef KX_TK
}

// one workgroup, thread e owns expert e: count, exclusive scan, stable placement.
// pair_work, if set, receives a second work list with one record per pair, {expert, q, q + 1, pairs[q]} for sorted
// pair q: the routed kernels then give every (chunk, pair) a workgroup of its own, and the workgroups of one chunk
// (an expert's pairs are neighbours in the list, so they are `chunks per expert` apart in the grid) stream it at the
// same time instead of one workgroup streaming it once per pair.
// The ids are staged in LDS (padded with 0xffff to a multiple of 8) and scanned 8 at a time;
// `staged` says the caller has already put them there.
__device__ __forceinline__ void bucket_block(const uint16_t *__restrict__ ids, int n_pairs, int E,
                                             int *__restrict__ counts, int *__restrict__ offsets,
                                             int *__restrict__ pairs, int4 *__restrict__ work,
                                             int *__restrict__ n_active, uint4 *s_ids4, int *s_cnt, int *s_act,
                                             bool staged = false, int4 *__restrict__ pair_work = nullptr) {
  const int e = threadIdx.x, n = blockDim.x;
  const int n8 = (n_pairs + 7) >> 3;
  uint16_t *s_ids = (uint16_t *)s_ids4;
  if (!staged) {
    for (int p = threadIdx.x; p < n8 * 8; p += n) s_ids[p] = p < n_pairs ? ids[p] : (uint16_t)0xffff;
    __syncthreads();
  }
  const uint32_t me = (uint32_t)e, me2 = me | (me << 16);
  int cnt = 0, off, slot, total_active, total;
  if (n_pairs <= 64) {
    // Few pairs (decode steps of up to 8 tokens): every thread goes over the pairs itself.  Expert e's offset is the
    // number of pairs with a smaller id and its slot the number of distinct smaller ids, so no scan over the
    // workgroup is needed (18 barriers at 448 threads); s_act[q] marks the first pair of each id.
    if (e < n8 * 8) {
      const uint16_t id = s_ids[e];
      int first = e < n_pairs;
      for (int q = 0; q < e; ++q) first &= s_ids[q] != id;
      s_act[e] = first;
    }
    __syncthreads();
    off = slot = total_active = 0;
    for (int q = 0; q < n_pairs; ++q) {
      const uint32_t id = s_ids[q];
      const int f = s_act[q];
      cnt += id == me;
      off += id < me;
      slot += f && id < me;
      total_active += f;
    }
    total = n_pairs;
  } else {
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
    off = s_cnt[e] - cnt;
    slot = s_act[e] - (cnt > 0 ? 1 : 0);
    total_active = s_act[n - 1];
    total = s_cnt[n - 1];
  }
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
            if (pair_work) pair_work[pos] = make_int4(e, pos, pos + 1, q * 8 + j);
            pairs[pos++] = q * 8 + j;
          }
        }
      }
    if (cnt > 0) work[slot] = make_int4(e, off, off + cnt, first);
    if (e >= total_active) work[e] = make_int4(-1, 0, 0, 0);
  }
  if (e == 0) {
    offsets[E] = total;
    *n_active = total_active;
  }
}

// Bucketing of up to 32 tokens whose ids are distinct within a token (what the top-k gives): one bit per expert and
// token, so an expert's count and a pair's place among its expert's pairs are population counts, and no thread goes
// over all pairs (bucket_block at 256 pairs: 15 us of the 384 threads each scanning them twice).  The results are
// bucket_block's.  A workgroup of at least E threads, a multiple of 64 and at most 1024; s_mask and s_pos: E ints each.
__device__ __forceinline__ void bucket_masks(const uint16_t *s_ids, int tokens, int topk, int E, int *__restrict__ counts,
                                             int *__restrict__ offsets, int *__restrict__ pairs, int4 *__restrict__ work,
                                             int *__restrict__ n_active, int *s_mask, int *s_pos,
                                             int4 *__restrict__ pair_work) {
  __shared__ int s_wave[2][16];
  const int tid = threadIdx.x, n = blockDim.x, n_pairs = tokens * topk;
  for (int e = tid; e < E; e += n) s_mask[e] = 0;
  __syncthreads();
  for (int p = tid; p < n_pairs; p += n) atomicOr((unsigned *)&s_mask[s_ids[p]], 1u << (p / topk));
  __syncthreads();
  const unsigned m = tid < E ? (unsigned)s_mask[tid] : 0u;
  const int cnt = __popc(m), act = cnt > 0 ? 1 : 0;
  // exclusive scans of counts and of the experts with work: inside the wave by shuffles, across the waves by their totals
  int sc = cnt, sa = act;
  const int lane = tid & 63, wave = tid >> 6, waves = n >> 6;
  for (int d = 1; d < 64; d <<= 1) {
    const int a = __shfl_up(sc, d), b = __shfl_up(sa, d);
    if (lane >= d) {
      sc += a;
      sa += b;
    }
  }
  if (lane == 63) {
    s_wave[0][wave] = sc;
    s_wave[1][wave] = sa;
  }
  __syncthreads();
  int base_c = 0, base_a = 0, total = 0, total_active = 0;
  for (int w = 0; w < waves; ++w) {
    const int c = s_wave[0][w], a = s_wave[1][w];
    if (w < wave) {
      base_c += c;
      base_a += a;
    }
    total += c;
    total_active += a;
  }
  const int off = base_c + sc - cnt, slot = base_a + sa - act;
  if (tid < E) {
    counts[tid] = cnt;
    offsets[tid] = off;
    s_pos[tid] = off | (slot << 16);
    if (tid >= total_active) work[tid] = make_int4(-1, 0, 0, 0);
  }
  if (tid == 0) {
    offsets[E] = total;
    *n_active = total_active;
  }
  __syncthreads();
  for (int p = tid; p < n_pairs; p += n) {
    const int id = s_ids[p], t = p / topk;
    const unsigned mm = (unsigned)s_mask[id];
    const int rank = __popc(mm & ((1u << t) - 1u));
    const int po = s_pos[id], o = po & 0xffff, pos = o + rank;
    pairs[pos] = p;
    if (pair_work) pair_work[pos] = make_int4(id, pos, pos + 1, p);
    if (rank == 0) work[po >> 16] = make_int4(id, o, o + __popc(mm), p);
  }
}

// top-k of `tokens` tokens (wave w takes tokens w, w + waves, ...), then the bucketing, by one workgroup
// of at least E threads.  s_ids4 holds ceil(tokens * topk / 8) pieces; s_cnt and s_act blockDim ints each.
// MASKS: more than 64 pairs of up to 32 tokens are bucketed by bucket_masks.
template <int EPL, bool COHERENT = false, bool MASKS = false>
__device__ __forceinline__ void route_block(const float *__restrict__ logits, const float *__restrict__ bias,
                                            uint16_t *__restrict__ ids, float *__restrict__ weights, int tokens, int E,
                                            int topk, float routed_scale, int *__restrict__ counts,
                                            int *__restrict__ offsets, int *__restrict__ pairs, int4 *__restrict__ work,
                                            int *__restrict__ n_active, uint4 *s_ids4, int *s_cnt, int *s_act,
                                            int4 *__restrict__ pair_work = nullptr) {
  uint16_t *s_ids = (uint16_t *)s_ids4;
  const int n_pairs = tokens * topk, n8 = (n_pairs + 7) >> 3;
  for (int p = n_pairs + threadIdx.x; p < n8 * 8; p += blockDim.x) s_ids[p] = (uint16_t)0xffff;
  const int wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  for (int t = wave; t < tokens; t += waves)
    topk_token<EPL, COHERENT>(logits + (size_t)t * E, bias, ids + (size_t)t * topk, weights + (size_t)t * topk, E, topk,
                              routed_scale, threadIdx.x & 63, s_ids + t * topk);
  __syncthreads();
  if (MASKS && n_pairs > 64 && tokens <= 32 && n_pairs < 65536 && (blockDim.x & 63) == 0)
    bucket_masks(s_ids, tokens, topk, E, counts, offsets, pairs, work, n_active, s_cnt, s_act, pair_work);
  else
    bucket_block(ids, n_pairs, E, counts, offsets, pairs, work, n_active, s_ids4, s_cnt, s_act, true, pair_work);
}

// route_block with the per-lane expert count chosen at run time; COHERENT: the logits were written by other
// workgroups of the same launch and are read with device-scope loads
template <bool COHERENT = false>
__device__ __forceinline__ void route_block_any(const float *logits, const float *bias, uint16_t *ids, float *weights,
                                                int tokens, int E, int topk, float routed_scale, int *counts, int *offsets,
                                                int *pairs, int4 *work, int *n_active, uint4 *s_ids4, int *s_cnt, int *s_act,
                                                int4 *pair_work = nullptr) {
  const int epl = (E + 63) >> 6;
#define KX_RB(N) route_block<N, COHERENT>(logits, bias, ids, weights, tokens, E, topk, routed_scale, counts, offsets, pairs, work, n_active, s_ids4, s_cnt, s_act, pair_work)
  if (epl <= 1) KX_RB(1);
  else if (epl <= 2) KX_RB(2);
  else if (epl <= 4) KX_RB(4);
  else if (epl <= 6) KX_RB(6);
  else if (epl <= 8) KX_RB(8);
  else KX_RB(16);
#undef KX_RB
}

}  // namespace kxr
