// kx_attn_parts.h -- the small steps between the attention projections, as device functions shared by the
// stand-alone kernel (q_absorb_k, kx_mla.hip) and by the q_b GEMV that finishes them in its own launch
// (gemv_absorb_k, kx_dense.hip): kv_a RMSNorm + RoPE of the shared key + cache write, and
// q_abs[t][h] = (bf(W_UK[h]^T q_nope[h]) | rope(q_rope[h])).
//
// Reference: src/kimi_exec.cu:817-824 (kv_a norm, rope_k :346-357, cache write), :818 (kv_b as W_UK).
#pragma once
#include "kx_common.h"
#include "kx_gemv_body.h"
#include "kx_math.h"
#include "kx_wave.h"

// seqs (stand-alone q absorb kernel only): 0: token t is sequence t at position pos.  n > 0 (a prefill step of several
// positions of n sequences): token t = i * n + b is position pos + i of sequence b; rope_row then points at the row of
// position pos, the rows of the following positions behind it.
struct QAbsArgs {
  const uint16_t *q, *kvb, *rope_row;
  float *qabs;
  const uint16_t *kva, *w_kv_ln;  // kva: first kv_a output row, kva_stride elements between tokens
  uint16_t *cache;
  size_t seq_stride;
  int heads, nope, rope, v_head, kv_rank, kva_stride, pos;
  float eps;
  int *head_count;  // gemv_absorb_k only: one counter per head, zero before the launch and left at zero
  int head_chunks;  // gemv_absorb_k only: workgroups per head
  int seqs;         // q_absorb_k only, see above
};

namespace kxa {

using kxg::unpack8;

// RMSNorm of one row by the first 256 threads of a workgroup; the schedule of rmsnorm_k (kx_dense.hip).
// Every thread of the workgroup must call it (it contains barriers).  A workgroup of fewer than 256
// threads must cover the row's n/8 chunks with one chunk per thread (the missing waves add +0).
__device__ __forceinline__ void rmsnorm_block(const uint16_t *xr, const uint16_t *w, uint16_t *yr, int n, float eps,
                                              float *ws /* 4 floats of LDS */) {
  const int chunks = n >> 3;
  const bool active = threadIdx.x < 256;
  float v = 0.0f;
  if (active)
    for (int c = threadIdx.x; c < chunks; c += 256) {
      float f[8];
      unpack8(f, ((const uint4 *)xr)[c]);
#pragma unroll
      for (int e = 0; e < 8; ++e) v = __builtin_fmaf(f[e], f[e], v);
    }
  float vv[1] = {v};
  kxw::reduce<1, 64>(vv, threadIdx.x & 63);
  __syncthreads();  // ws may still be read from a previous call
  if (threadIdx.x < 4) ws[threadIdx.x] = 0.0f;
  __syncthreads();
  if (active && (threadIdx.x & 63) == 0) ws[threadIdx.x >> 6] = vv[0];
  __syncthreads();
  const float total = ((ws[0] + ws[1]) + ws[2]) + ws[3];
  const float scale = kx_rsqrtf(total / (float)n + eps);
  if (active)
    for (int c = threadIdx.x; c < chunks; c += 256) {
      float f[8], g[8];
      unpack8(f, ((const uint4 *)xr)[c]);
      unpack8(g, ((const uint4 *)w)[c]);
      uint32_t o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        uint32_t a = kx_bf16_rne(kx_bfround(f[2 * e] * scale) * g[2 * e]);
        uint32_t b = kx_bf16_rne(kx_bfround(f[2 * e + 1] * scale) * g[2 * e + 1]);
        o[e] = a | (b << 16);
      }
      ((uint4 *)yr)[c] = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// interleaved-pair rotation of rope_k (:352-356): reads (2p, 2p+1), writes (p, half+p)
__device__ __forceinline__ void rope_pair(float x0, float x1, float c, float s, float &y_lo, float &y_hi) {
  y_lo = kx_bfround(kx_bfround(x0 * c) - kx_bfround(x1 * s));
  y_hi = kx_bfround(kx_bfround(x1 * c) + kx_bfround(x0 * s));
}

// kv_a RMSNorm on the latent part only (:817), RoPE of the shared rope key (:820-823) and the write of
// the cache row (:824) for token t; kva bf16 [kv_rank + rope] is the kv_a output of the token.
__device__ __forceinline__ void kv_finish_block(const uint16_t *kva, const uint16_t *w_kv_ln, const uint16_t *rope_row,
                                                uint16_t *crow, int kv_rank, int rope, float eps, float *ws) {
  rmsnorm_block(kva, w_kv_ln, crow, kv_rank, eps, ws);
  const int half = rope >> 1;
  if ((int)threadIdx.x < half) {
    const int p = threadIdx.x;
    const uint16_t *kr = kva + kv_rank;
    float lo, hi;
    rope_pair(kx_bf16_f32(kr[2 * p]), kx_bf16_f32(kr[2 * p + 1]), kx_bf16_f32(rope_row[p]), kx_bf16_f32(rope_row[half + p]),
              lo, hi);
    crow[kv_rank + p] = kx_bf16_rne(lo);
    crow[kv_rank + half + p] = kx_bf16_rne(hi);
  }
}

// q_abs of head h for `tokens` tokens by one whole workgroup, from q rows that other workgroups of the same
// launch have just stored with device-scope stores (read here with device-scope loads).  The sums are those of
// q_absorb_k: for every latent column eight fma chains over d = j, j+8, ..., then ((0+1)+(2+3))+((4+5)+(6+7)).
// Thread item (chain, column group of 8) = (i / (kv_rank/8), i % (kv_rank/8)), so a wave reads whole rows of W_UK.
// part: LDS [8][kv_rank] floats, qs: LDS [nope + rope] floats.  Contains barriers: every thread must call it.
__device__ __forceinline__ void absorb_head_block(const QAbsArgs &a, int h, int tokens, float *part, float *qs) {
  const int nope = a.nope, rope = a.rope, kv_rank = a.kv_rank;
  const int qk = nope + rope, kva = kv_rank + rope, half = rope >> 1;
  const int ncg = kv_rank >> 3;
  const uint16_t *wuk = a.kvb + (size_t)h * (nope + a.v_head) * kv_rank;
  for (int t = 0; t < tokens; ++t) {
    const uint32_t *qh = (const uint32_t *)(a.q + ((size_t)t * a.heads + h) * qk);
    float *out = a.qabs + ((size_t)t * a.heads + h) * kva;
    for (int i = threadIdx.x; i < (qk >> 1); i += blockDim.x) {
      const uint32_t u = kx_arrive_load(qh + i);
      qs[2 * i] = kxg::bf_lo(u);
      qs[2 * i + 1] = kxg::bf_hi(u);
    }
    __syncthreads();
    for (int item = threadIdx.x; item < 8 * ncg; item += blockDim.x) {
      const int chain = item / ncg, cg = item - chain * ncg;
      float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 8
      for (int d = chain; d < nope; d += 8) {
        float wf[8];
        unpack8(wf, *(const uint4 *)(wuk + (size_t)d * kv_rank + cg * 8));
        const float qd = qs[d];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(wf[e], qd, acc[e]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) part[chain * kv_rank + cg * 8 + e] = acc[e];
    }
    __syncthreads();
    for (int c = threadIdx.x; c < kv_rank; c += blockDim.x) {
      const float *p = part + c;
      const float s = ((p[0] + p[kv_rank]) + (p[2 * kv_rank] + p[3 * kv_rank])) +
                      ((p[4 * kv_rank] + p[5 * kv_rank]) + (p[6 * kv_rank] + p[7 * kv_rank]));
      out[c] = kx_bfround(s);
    }
    if ((int)threadIdx.x < half) {
      const int p = threadIdx.x;
      float lo, hi;
      rope_pair(qs[nope + 2 * p], qs[nope + 2 * p + 1], kx_bf16_f32(a.rope_row[p]), kx_bf16_f32(a.rope_row[half + p]), lo, hi);
      out[kv_rank + p] = lo;
      out[kv_rank + half + p] = hi;
    }
    __syncthreads();  // part and qs are reused by the next token
  }
}

}  // namespace kxa
