// kx_dense.hip -- RMSNorm and the bf16-weight GEMV family (attention projections,
// router gate, shared expert, dense MLP, lm_head) for T activation rows.
//
// Reference: rmsnorm_k (src/kimi_exec.cu:258-270), matvec_bf16_k (:272-284),
// matvec_bf16_f32_k (:286-298), silu_mul_k (:253-256), add_k (:248-251),
// expert_accum_k / round_bf16_k (:399-407), argmax_k (:477-493).  The
// reference runs one 256-thread block per output row over NVMe-streamed
// 64-row tiles; here a wave owns a 512-column slice of the rows of a work item
// (one 1 KB contiguous read per row), keeps its 8 activations per token in
// registers, and the elementwise kernels above are epilogues of the GEMV.
//
// Summation order of y[t, r] (fixed, independent of T):
//   lane partial  p[s][l] = fma chain over e = 0..7 of w[r, 512 s + 8 l + e] * x[t, ...]
//   slice sum     B[s]    = xor-butterfly over the 64 lanes (32,16,8,4,2,1)
//   row sum       y       = B[0] + B[1] + ... + B[S-1], left to right
#include <mutex>
#include "kx_arrive.h"
#include "kx_attn_parts.h"
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_gemv_body.h"
#include "kx_math.h"
#include "kx_route.h"
#include "kx_wave.h"

namespace {

using namespace kxg;

// ---- RMSNorm ----------------------------------------------------------------------
// one 256-thread workgroup per row; thread t owns 8-element chunks t, t+256, ...
__global__ void __launch_bounds__(256) rmsnorm_k(const uint16_t *__restrict__ x, const uint16_t *__restrict__ w,
                                                 uint16_t *__restrict__ y, int n, int x_stride, int y_stride,
                                                 float eps) {
  __shared__ float ws[4];
  const uint16_t *xr = x + (size_t)blockIdx.x * x_stride;
  uint16_t *yr = y + (size_t)blockIdx.x * y_stride;
  const int chunks = n >> 3;
  float v = 0.0f;
  for (int c = threadIdx.x; c < chunks; c += 256) {
    float f[8];
    unpack8(f, ((const uint4 *)xr)[c]);
#pragma unroll
    for (int e = 0; e < 8; ++e) v = __builtin_fmaf(f[e], f[e], v);
  }
  float vv[1] = {v};
  kxw::reduce<1, 64>(vv, threadIdx.x & 63);
  if ((threadIdx.x & 63) == 0) ws[threadIdx.x >> 6] = vv[0];
  __syncthreads();
  float total = ((ws[0] + ws[1]) + ws[2]) + ws[3];
  float scale = kx_rsqrtf(total / (float)n + eps);
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

template <int MATS, int RI, int TT>
__global__ void __launch_bounds__(TT > 1 ? 512 : 1024) gemv_bf16_k(KxGemvArgs a) {
  extern __shared__ float part[];
  gemv_body<MATS, RI, TT>(a, blockIdx.x, gridDim.x, part);
}

// The same GEMV with the tokens spread over the grid: workgroup (c, y) takes chunk c for tokens 4 y .. 4 y + 3.  For
// many tokens against a small matrix (router logits, the per-head W_UV blocks): one workgroup going over the token
// blocks one after the other spends its time waiting for each block's activations, while the weights all these
// workgroups read again come from L2.  The sums are those of gemv_bf16_k (they do not depend on the launch shape).
template <int RI>
__global__ void __launch_bounds__(512) gemv_tokblk_k(KxGemvArgs a) {
  extern __shared__ float part[];
  const int t0 = blockIdx.y * 4;
  a.x += (size_t)t0 * a.x_stride;
  a.out = (char *)a.out + (size_t)t0 * a.out_stride * (a.epi == KX_EPI_F32 ? 4 : 2);
  a.tokens = min(4, a.tokens - t0);
  gemv_body<1, RI, 4>(a, blockIdx.x, gridDim.x, part);
}

// Two GEMVs over the same activations in one launch: the first gridDim.x - n0 workgroups run the
// second problem (the router gate, f32 logits), the other n0 the first (two matrices, SwiGLU:
// the shared expert's gate and up).  The router workgroup that finishes last routes the tokens: top-k and
// bucketing, from the logits that all of them have written by then.
struct KxRouteArgs {
  int *counter;  // zero before the launch; the routing workgroup leaves it at zero
  const float *bias;
  uint16_t *ids;
  float *weights;
  int experts, topk;
  float routed_scale;
  int *counts, *offsets, *pairs;
  int4 *work;
  int *n_active;
  int4 *pair_work;  // optional second work list, one record per pair
};
// gemv_tokblk_k for the router's logits of 8 to 32 tokens that also routes them, in two steps of "the last one in
// finishes the job": the workgroup that completes a block of four tokens does their top-k (a wave per token), and
// the one of those that comes last buckets all tokens (kxr::bucket_masks).  r.counter: 1 + gridDim.y ints, zero
// before the launch and left at zero.
template <int RI>
__global__ void __launch_bounds__(512) gemv_tokblk_route_k(KxGemvArgs a, KxRouteArgs r) {
  extern __shared__ float part[];
  __shared__ int s_last;
  __shared__ int s_mask[512];
  __shared__ int s_pos[512];
  __shared__ uint16_t s_ids[1024];
  const int tokens = a.tokens, t0 = blockIdx.y * 4, nt = min(4, tokens - t0);
  const float *logits = (const float *)a.out + (size_t)t0 * a.out_stride;
  const int stride = a.out_stride;
  a.x += (size_t)t0 * a.x_stride;
  a.out = (float *)a.out + (size_t)t0 * a.out_stride;
  a.tokens = nt;
  gemv_body<1, RI, 4>(a, blockIdx.x, gridDim.x, part);
  kx_arrive_writes_done();
  __syncthreads();
  if (threadIdx.x == 0) s_last = kx_arrive_is_last(r.counter + 1 + blockIdx.y, gridDim.x);
  __syncthreads();
  if (!s_last) return;
  const int wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  for (int t = wave; t < nt; t += waves)
    kxr::topk_token_any<true, true>(logits + (size_t)t * stride, r.bias, r.ids + (size_t)(t0 + t) * r.topk,
                                    r.weights + (size_t)(t0 + t) * r.topk, r.experts, r.topk, r.routed_scale, threadIdx.x & 63);
  if (threadIdx.x == 0) kx_arrive_reset(r.counter + 1 + blockIdx.y);
  kx_arrive_writes_done();
  __syncthreads();  // also: every thread has read s_last before it is written again
  if (threadIdx.x == 0) s_last = kx_arrive_is_last(r.counter, gridDim.y);
  __syncthreads();
  if (!s_last) return;
  const int n_pairs = tokens * r.topk;
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) s_ids[p] = kx_arrive_load(r.ids + p);
  __syncthreads();
  kxr::bucket_masks(s_ids, tokens, r.topk, r.experts, r.counts, r.offsets, r.pairs, r.work, r.n_active, s_mask, s_pos, r.pair_work);
  if (threadIdx.x == 0) kx_arrive_reset(r.counter);
}

template <int RI0, int RI1, int TT>
__global__ void __launch_bounds__(TT > 1 ? 512 : 1024) gemv_pair_k(KxGemvArgs a0, KxGemvArgs a1, int n0, KxRouteArgs r) {
  extern __shared__ float part[];
  const int n1 = gridDim.x - n0;  // the router's workgroups come first: its routing tail overlaps the rest
  if ((int)blockIdx.x >= n1) {
    gemv_body<2, RI0, TT>(a0, blockIdx.x - n1, n0, part);
    return;
  }
  gemv_body<1, RI1, TT>(a1, blockIdx.x, n1, part);
  if (!r.counter) return;
  __shared__ int s_last;
  __shared__ int s_cnt[1024];
  __shared__ int s_act[1024];
  __shared__ uint4 s_ids4[4];
  // The logits were stored with device-scope stores; after the barrier one thread counts the workgroup in
  // (release).  The workgroup that counts in last (acquire) reads all logits with device-scope loads.
  kx_arrive_writes_done();
  __syncthreads();
  if (threadIdx.x == 0) s_last = kx_arrive_is_last(r.counter, n1);
  __syncthreads();
  if (!s_last) return;
  kxr::route_block_any<true>((const float *)a1.out, r.bias, r.ids, r.weights, a1.tokens, r.experts, r.topk, r.routed_scale,
                       r.counts, r.offsets, r.pairs, r.work, r.n_active, s_ids4, s_cnt, s_act, r.pair_work);
  if (threadIdx.x == 0) kx_arrive_reset(r.counter);
}

// The q_b GEMV that also finishes the query.  Workgroup 0 norms kv_a, rotates the shared rope key and writes the
// cache row; workgroup 1 + c computes chunk c of q (device-scope stores) and counts itself in on the counter of
// its head; the one that counts in last has all of the head's q in memory and computes q_abs of the head (W_UK
// absorb + RoPE) while other heads are still streaming.  Nothing waits for another workgroup.
template <int RI, int TT>
__global__ void __launch_bounds__(TT > 1 ? 512 : 1024) gemv_absorb_k(KxGemvArgs a, QAbsArgs q) {
  extern __shared__ float part[];
  __shared__ float ab_part[8 * 512];
  __shared__ float ab_q[256];
  __shared__ float ab_ws[4];
  __shared__ int s_last;
  // The cache row is the first workgroup's job: its dependent loads are answered fast while the launch is young (the
  // same job given to the last workgroup, which starts once the memory pipeline is full, made the launch 2 us longer).
  if (blockIdx.x == 0) {
    const int kva = q.kv_rank + q.rope;
    for (int t = 0; t < a.tokens; ++t)
      kxa::kv_finish_block(q.kva + (size_t)t * q.kva_stride, q.w_kv_ln, q.rope_row,
                           q.cache + (size_t)t * q.seq_stride + (size_t)q.pos * kva, q.kv_rank, q.rope, q.eps, ab_ws);
    return;
  }
  const int chunk = blockIdx.x - 1;
  gemv_body<1, RI, TT>(a, chunk, gridDim.x - 1, part);
  kx_arrive_writes_done();
  __syncthreads();  // every lane's stores of q lie before the counting lane's release (kx_arrive.h)
  const int h = chunk / q.head_chunks;
  if (threadIdx.x == 0) s_last = kx_arrive_is_last(q.head_count + h, q.head_chunks);
  __syncthreads();
  if (!s_last) return;
  kxa::absorb_head_block(q, h, a.tokens, ab_part, ab_q);
  if (threadIdx.x == 0) kx_arrive_reset(q.head_count + h);
}

// lowest-index argmax over bf16-rounded logits (sample_lm_head :718-734, argmax_k :477-493), in two
// stages: ARGMAX_PARTS workgroups per row each reduce a slice, then one wave per row merges them
constexpr int ARGMAX_PARTS = 64;

__device__ __forceinline__ void argmax_merge(float &best, uint32_t &bi, float ov, uint32_t oi) {
  if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
}
__device__ __forceinline__ void argmax_wave(float &best, uint32_t &bi) {
  for (int m = 32; m; m >>= 1) {
    float ov = __shfl_xor(best, m);
    uint32_t oi = (uint32_t)__shfl_xor((int)bi, m);
    argmax_merge(best, bi, ov, oi);
  }
}

__global__ void __launch_bounds__(256) argmax_part_k(const float *__restrict__ logits, int n, int stride,
                                                     float *__restrict__ pv, uint32_t *__restrict__ pi) {
  __shared__ float sv[4];
  __shared__ uint32_t si[4];
  const float *p = logits + (size_t)blockIdx.y * stride;
  const int per = (n + ARGMAX_PARTS - 1) / ARGMAX_PARTS;
  const int lo = blockIdx.x * per, hi = min(n, lo + per);
  float best = -__builtin_inff();
  uint32_t bi = 0xffffffffu;
  for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
    float v = p[i];
    if (v > best) { best = v; bi = (uint32_t)i; }
  }
  argmax_wave(best, bi);
  if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) argmax_merge(best, bi, sv[w], si[w]);
    pv[blockIdx.y * ARGMAX_PARTS + blockIdx.x] = best;
    pi[blockIdx.y * ARGMAX_PARTS + blockIdx.x] = bi;
  }
}
__global__ void __launch_bounds__(64) argmax_final_k(const float *__restrict__ pv, const uint32_t *__restrict__ pi,
                                                     uint32_t *__restrict__ out) {
  float best = pv[blockIdx.x * ARGMAX_PARTS + threadIdx.x];
  uint32_t bi = pi[blockIdx.x * ARGMAX_PARTS + threadIdx.x];
  argmax_wave(best, bi);
  if (threadIdx.x == 0) out[blockIdx.x] = bi == 0xffffffffu ? 0u : bi;  // every logit -inf or NaN: id 0 as :481
}

template <int MATS, int RI>
void launch_tt(const KxGemvArgs &a, int tt, dim3 g, dim3 b, size_t lds, hipStream_t st) {
  if constexpr (RI * MATS * 4 <= 16) {
    if (tt >= 4) { hipLaunchKernelGGL((gemv_bf16_k<MATS, RI, 4>), g, b, lds, st, a); return; }
  }
  if constexpr (RI * MATS * 2 <= 16) {
    if (tt >= 2) { hipLaunchKernelGGL((gemv_bf16_k<MATS, RI, 2>), g, b, lds, st, a); return; }
  }
  hipLaunchKernelGGL((gemv_bf16_k<MATS, RI, 1>), g, b, lds, st, a);
}

template <int MATS>
void launch_ri(const KxGemvArgs &a, int ri, int tt, dim3 g, dim3 b, size_t lds, hipStream_t st) {
  if constexpr (MATS == 1) {
    if (ri == 4) { launch_tt<MATS, 4>(a, tt, g, b, lds, st); return; }
  }
  if (ri >= 2) launch_tt<MATS, 2>(a, tt, g, b, lds, st);
  else launch_tt<MATS, 1>(a, tt, g, b, lds, st);
}

}  // namespace

namespace {
// Fills in the launch shape of a GEMV (a.epi, a.nw, a.rs, a.nt) and returns rows per wave and tile in
// ri; ri_max caps it.  Returns the rows per chunk, or -1 after setting the error.
int gemv_plan(int epi, KxGemvArgs &a, int &ri, int ri_max, int target_chunks = 256) {
  if (!(a.cols > 0 && a.cols % 512 == 0)) { kx_set_error("kx_gemv: cols=%d must be a positive multiple of 512", a.cols); return -1; }
  if (!(a.rows > 0 && a.tokens > 0)) { kx_set_error("kx_gemv: rows=%d tokens=%d must be positive", a.rows, a.tokens); return -1; }
  if (!(epi >= KX_EPI_BF16 && epi <= KX_EPI_ARGMAX)) { kx_set_error("kx_gemv: unknown epilogue %d", epi); return -1; }
  const int S = a.cols / 512;
  const int mats = epi == KX_EPI_SWIGLU ? 2 : 1;
  a.epi = epi;
  // waves per workgroup: the largest divisor of S up to 8 (even slice counts per wave),
  // times row sets to reach 8 waves
  a.nw = 1;
  for (int d = 2; d <= 8; ++d)
    if (S % d == 0) a.nw = d;
  a.rs = 8 / a.nw;
  // 3, 5 or 6 slice waves leave the workgroup short of 8 waves (6, 5, 6; 7 slice waves are 7), and a wave that goes through its tiles one
  // load latency at a time then has too little in flight for the CU: twice the row sets (12, 10, 12 waves).  The q_b
  // GEMV (1536 columns) goes through six tiles per wave.
  if ((a.nw == 3 || a.nw == 5 || a.nw == 6) && a.tokens == 1) a.rs *= 2;  // one token: the kernels that take 1024 threads
  while (a.rs > 1 && a.rs > a.rows) a.rs >>= 1;
  // rows per wave and tile, tiles per chunk: a few hundred chunks when the matrix allows
  ri = a.rows >= 2048 * a.rs ? 4 : a.rows >= 768 * a.rs ? 2 : 1;
  // From two tokens on the chunks are made for one round of workgroups anyway (below), and a wave spends a load's
  // latency on every tile: four rows per tile whatever the matrix (q_a|kv_a at four tokens: 10 steps of two rows per
  // wave, 23 us; W_UV the same).
  if (a.tokens >= 2 && !(a.row_block && a.row_block % (4 * a.rs))) ri = 4;
  while (ri > 1 && ri * a.rs > a.rows) ri >>= 1;
  if (ri * mats > 4) ri = 4 / mats;
  if (ri > ri_max) ri = ri_max;
  const int rt = a.rs * ri;
  int nt = a.rows / (rt * target_chunks);
  // From two tokens on a CU holds one workgroup of these kernels, not two (150-210 registers against 128): more chunks
  // than CUs would be a second round of a few workgroups, so the chunks are made long enough for one round where
  // eight tiles allow it.  (Twice the rows per tile on top of that, to put a one-token launch's bytes in flight per CU,
  // changed nothing.)
  if (a.tokens >= 2) nt = kx_cdiv(a.rows, rt * (target_chunks < 256 ? target_chunks : 256));
  nt = nt < 1 ? 1 : nt > 8 ? 8 : nt;
  // One token: a CU holds two workgroups, and a plan that gives a few more chunks than CUs (q_a|kv_a at Kimi shapes:
  // 264) leaves a few CUs with twice the bytes of the rest: one more tile per chunk (176 chunks; 250.3 -> 250.9 tok/s).
  if (a.tokens == 1 && nt < 8) {
    const int chunks = kx_cdiv(a.rows, rt * nt);
    if (chunks > 256 && chunks <= 320) ++nt;
  }
  if (a.row_block) {  // a chunk must not straddle blocks
    if (!(a.rows % a.row_block == 0 && a.row_block % rt == 0)) { kx_set_error("kx_gemv: row_block=%d does not fit tiles of %d rows", a.row_block, rt); return -1; }
    while (a.row_block % (rt * nt)) --nt;
  }
  a.nt = nt;
  if (a.norm_w && !(a.tokens <= 4 && a.nw * a.rs * 64 >= 256 && !a.row_block)) {
    kx_set_error("kx_gemv: the fused RMSNorm needs at most 4 tokens and 256 threads");
    return -1;
  }
  if (a.mla_po) {
    if (!(a.row_block && a.cols == 512 && !a.norm_w)) { kx_set_error("kx_gemv: attention partials feed a 512-column blocked matrix"); return -1; }
    if (!(a.tokens <= 4 && a.mla_spans >= 1 && a.mla_spans <= 64)) {
      kx_set_error("kx_gemv: the fused attention merge takes at most 4 tokens and 64 spans (got %d, %d)", a.tokens, a.mla_spans);
      return -1;
    }
  }
  return rt * nt;
}
}  // namespace

int kx_gemv_plan(int epi, KxGemvArgs &a, int *ri) { return gemv_plan(epi, a, *ri, 4); }

// Tokens are taken in blocks of at most 32 (LDS holds a partial per token and slice).
// route, routed: the router's logits; *routed says whether the launch has also done the routing (gemv_tokblk_route_k)
static int gemv_launch_impl(int epi, KxGemvArgs a, hipStream_t st, const KxRouteArgs *route, bool *routed) {
  int ri;
  const int CR = gemv_plan(epi, a, ri, 4);
  if (CR < 0) return KX_ERR_ARG;
  const int S = a.cols / 512;
  const int mats = epi == KX_EPI_SWIGLU ? 2 : 1;
  const int all_tokens = a.tokens;
  const uint16_t *x0 = a.x;
  char *out0 = (char *)a.out;
  const size_t out_elem = (epi == KX_EPI_F32 || epi == KX_EPI_ARGMAX) ? 4 : 2;
  // 8 tokens and more against a matrix that stays in L2: the token blocks side by side (gemv_tokblk_k), all in one launch
  if (all_tokens >= 8 && all_tokens <= 4 * 65535 && (epi == KX_EPI_BF16 || epi == KX_EPI_F32) && !a.norm_w && !a.mla_po &&
      kx_cdiv(a.rows, CR) <= 4096 && (size_t)a.rows * a.cols * 2 <= (16u << 20)) {
    // A CU holds one workgroup of this kernel, and a wave spends a load's latency on every tile it goes through: one
    // round of workgroups (256 over the token blocks) and four rows per wave and tile, so that a chunk is a few steps
    // with four rows in flight per lane.  Longer chunks also divide the L2 traffic of the activations, which a chunk
    // reads once (one row per chunk: 57 KB of them against 14 KB of weights for the router).  The router at 32
    // tokens: 32 chunks of 12 rows in three steps per token block instead of 64 chunks of 6 rows in six steps and two
    // rounds.
    const int blocks = kx_cdiv(all_tokens, 4);
    KxGemvArgs b = a;
    int ri4;
    int CR4 = gemv_plan(epi, b, ri4, 4, 512 / blocks > 32 ? 512 / blocks : 32);
    if (CR4 < 0) return KX_ERR_ARG;
    {
      int r4 = 4;
      while (r4 > 1 && (r4 * b.rs > a.rows || (a.row_block && a.row_block % (r4 * b.rs)))) r4 >>= 1;
      const int rt = r4 * b.rs;
      const int per_block = 256 / blocks > 1 ? 256 / blocks : 1;
      int nt = kx_cdiv(kx_cdiv(a.rows, per_block), rt);
      nt = nt < 1 ? 1 : nt > 8 ? 8 : nt;
      if (a.row_block && a.row_block % rt == 0)
        while (a.row_block % (rt * nt)) --nt;
      if (rt * nt <= a.rows && (!a.row_block || a.row_block % rt == 0) && (size_t)rt * nt * 4 * S * sizeof(float) <= 64 * 1024) {
        ri4 = r4;
        b.nt = nt;
        CR4 = rt * nt;
      }
    }
    const size_t lds4 = (size_t)CR4 * 4 * S * sizeof(float);
    KX_REQUIRE(lds4 <= 64 * 1024, "kx_gemv: %zu bytes of LDS needed", lds4);
    const dim3 g(kx_cdiv(a.rows, CR4), blocks), blk(b.nw * b.rs * 64);
    const int threads = b.nw * b.rs * 64;
    if (route && epi == KX_EPI_F32 && all_tokens <= 32 && route->experts == a.rows && route->experts <= threads && threads <= 512 &&
        all_tokens * route->topk <= 1024 && route->topk <= 64 && route->topk <= route->experts && a.out_stride >= a.rows) {
      b.flags |= KX_GEMV_COHERENT_OUT;
      if (ri4 == 4) hipLaunchKernelGGL(gemv_tokblk_route_k<4>, g, blk, lds4, st, b, *route);
      else if (ri4 == 2) hipLaunchKernelGGL(gemv_tokblk_route_k<2>, g, blk, lds4, st, b, *route);
      else hipLaunchKernelGGL(gemv_tokblk_route_k<1>, g, blk, lds4, st, b, *route);
      KX_LAUNCH_CHECK();
      *routed = true;
      return KX_OK;
    }
    if (ri4 == 4) hipLaunchKernelGGL(gemv_tokblk_k<4>, g, blk, lds4, st, b);
    else if (ri4 == 2) hipLaunchKernelGGL(gemv_tokblk_k<2>, g, blk, lds4, st, b);
    else hipLaunchKernelGGL(gemv_tokblk_k<1>, g, blk, lds4, st, b);
    KX_LAUNCH_CHECK();
    return KX_OK;
  }
  for (int t0 = 0; t0 < all_tokens; t0 += 32) {
    a.tokens = all_tokens - t0 < 32 ? all_tokens - t0 : 32;
    a.x = x0 + (size_t)t0 * a.x_stride;
    a.out = out0 + (size_t)t0 * a.out_stride * out_elem;
    KxGemvArgs b = a;
    if (epi == KX_EPI_MOE_COMBINE) {
      b.expert_out = a.expert_out + (size_t)t0 * a.topk * a.rows;
      b.route_w = a.route_w + (size_t)t0 * a.topk;
    }
    const int tt = b.tokens >= 3 ? 4 : b.tokens >= 2 ? 2 : 1;
    const int chunks = kx_cdiv(a.rows, CR);
    const size_t lds = (size_t)mats * CR * b.tokens * S * sizeof(float);
    KX_REQUIRE(lds <= 160 * 1024, "kx_gemv: %zu bytes of LDS needed", lds);
    dim3 g(chunks < 4096 ? chunks : 4096), blk(a.nw * a.rs * 64);
    if (mats == 2) launch_ri<2>(b, ri, tt, g, blk, lds, st);
    else launch_ri<1>(b, ri, tt, g, blk, lds, st);
    KX_LAUNCH_CHECK();
  }
  return KX_OK;
}

int kx_gemv_launch(int epi, KxGemvArgs a, hipStream_t st) { return gemv_launch_impl(epi, a, st, nullptr, nullptr); }

int kx_gemv_route_launch(KxGemvArgs router, const float *bias, uint16_t *ids, float *weights, int experts, int topk,
                         float routed_scale, int *counts, int *offsets, int *pairs, int4 *work, int *n_active, int *counters,
                         bool *routed, hipStream_t st, int4 *pair_work) {
  KxRouteArgs r;
  r.counter = counters; r.bias = bias; r.ids = ids; r.weights = weights; r.experts = experts; r.topk = topk;
  r.routed_scale = routed_scale; r.counts = counts; r.offsets = offsets; r.pairs = pairs; r.work = work; r.n_active = n_active;
  r.pair_work = pair_work;
  *routed = false;
  return gemv_launch_impl(KX_EPI_F32, router, st, &r, routed);
}

// The shared expert's gate/up GEMV (SwiGLU epilogue) and the router's logits GEMV in one launch,
// with the routing (top-k, bucketing) done by the last router workgroup.  Returns KX_OK with
// *fused = false, having launched nothing, when the shapes do not allow the combination.
int kx_gemv_pair_route_launch(KxGemvArgs a0, KxGemvArgs a1, const float *bias, uint16_t *ids, float *weights, int experts,
                              int topk, float routed_scale, int *counts, int *offsets, int *pairs, int4 *work,
                              int *n_active, int *counter, bool *fused, hipStream_t st, int4 *pair_work) {
  *fused = false;
  if (a0.tokens != a1.tokens || a0.tokens > 4 || a0.tokens * topk > 32 || a0.cols != a1.cols || topk > 64 || topk > experts) return KX_OK;
  int ri0, ri1;
  int CR1 = gemv_plan(KX_EPI_F32, a1, ri1, 1, 128);
  if (CR1 < 0) return KX_ERR_ARG;
  // The routing waits for the last router workgroup, and a wave with one row per step spends a load's latency on every
  // step (three tiles of two slices at Kimi shapes: 6.4 us for 43 KB).  Four rows per step and one tile per chunk
  // where the rows allow: two steps.
  if (a1.rows % (a1.rs * 4) == 0 && !a1.row_block) {
    ri1 = 4;
    a1.nt = 1;
    CR1 = a1.rs * 4;
  }
  // from two tokens on the two parts share one round of workgroups (see gemv_plan)
  const int left = 256 - kx_cdiv(a1.rows, CR1);
  const int CR0 = gemv_plan(KX_EPI_SWIGLU, a0, ri0, 2, a0.tokens >= 2 && left >= 64 ? left : 256);
  if (CR0 < 0) return KX_ERR_ARG;
  const int threads = a0.nw * a0.rs * 64;
  if (threads != a1.nw * a1.rs * 64 || experts > threads || experts > 1024) return KX_OK;
  const int S = a0.cols / 512, T = a0.tokens;
  const size_t lds0 = (size_t)2 * CR0 * T * S * sizeof(float), lds1 = (size_t)CR1 * T * S * sizeof(float);
  const size_t lds = lds0 > lds1 ? lds0 : lds1;
  if (lds > 120 * 1024) return KX_OK;
  const int n0 = kx_cdiv(a0.rows, CR0), n1 = kx_cdiv(a1.rows, CR1);
  if (n0 + n1 > 4096) return KX_OK;
  KxRouteArgs r;
  r.counter = counter; r.bias = bias; r.ids = ids; r.weights = weights; r.experts = experts; r.topk = topk;
  a1.flags |= KX_GEMV_COHERENT_OUT;
  r.routed_scale = routed_scale; r.counts = counts; r.offsets = offsets; r.pairs = pairs; r.work = work; r.n_active = n_active; r.pair_work = pair_work;
  const int tt = T >= 3 ? 4 : T >= 2 ? 2 : 1;
  dim3 g(n0 + n1), blk(threads);
#define KX_PAIR(R, R1, TT_) hipLaunchKernelGGL((gemv_pair_k<R, R1, TT_>), g, blk, lds, st, a0, a1, n0, r)
#define KX_PAIR_TT(R, R1) do { if (tt == 4) KX_PAIR(R, R1, 4); else if (tt == 2) KX_PAIR(R, R1, 2); else KX_PAIR(R, R1, 1); } while (0)
  if (ri0 == 2) { if (ri1 == 4) KX_PAIR_TT(2, 4); else KX_PAIR_TT(2, 1); }
  else          { if (ri1 == 4) KX_PAIR_TT(1, 4); else KX_PAIR_TT(1, 1); }
#undef KX_PAIR_TT
#undef KX_PAIR
  KX_LAUNCH_CHECK();
  *fused = true;
  return KX_OK;
}

int kx_gemv_absorb_launch(KxGemvArgs g, const QAbsArgs &q0, bool *fused, hipStream_t st) {
  *fused = false;
  QAbsArgs q = q0;
  const int qk = q.nope + q.rope;
  if (g.tokens > 4 || g.rows != q.heads * qk || q.kv_rank > 512 || q.kv_rank % 8 || qk > 256 || qk % 2 || q.rope % 2 ||
      !q.head_count || !q.cache)
    return KX_OK;
  int ri;
  int CR = gemv_plan(KX_EPI_BF16, g, ri, 4, g.tokens >= 2 ? 255 : 256);  // one workgroup more writes the cache row
  if (CR < 0) return KX_ERR_ARG;
  while (qk % CR && g.nt < 16) CR = CR / g.nt * (g.nt + 1), ++g.nt;  // whole chunks per head
  const int threads = g.nw * g.rs * 64;
  if (qk % CR || g.rows / CR + 1 > 4096 || (threads < 256 && q.kv_rank / 8 > threads) || q.rope / 2 > threads) return KX_OK;
  q.head_chunks = qk / CR;
  g.flags |= KX_GEMV_COHERENT_OUT;
  const int S = g.cols / 512;
  const size_t lds = (size_t)CR * g.tokens * S * sizeof(float);
  KX_REQUIRE(lds <= 128 * 1024, "kx_gemv: %zu bytes of LDS needed", lds);
  const int tt = g.tokens >= 3 ? 4 : g.tokens >= 2 ? 2 : 1;
  dim3 grid(g.rows / CR + 1), blk(threads);
#define KX_ABS(R, TT_) hipLaunchKernelGGL((gemv_absorb_k<R, TT_>), grid, blk, lds, st, g, q)
#define KX_ABS_TT(R) do { if (tt == 4) KX_ABS(R, 4); else if (tt == 2) KX_ABS(R, 2); else KX_ABS(R, 1); } while (0)
  if (ri == 4) KX_ABS_TT(4);
  else if (ri >= 2) KX_ABS_TT(2);
  else KX_ABS_TT(1);
#undef KX_ABS_TT
#undef KX_ABS
  KX_LAUNCH_CHECK();
  *fused = true;
  return KX_OK;
}

int kx_rmsnorm_launch(const uint16_t *x, const uint16_t *w, uint16_t *y, int tokens, int n, int x_stride,
                      int y_stride, float eps, hipStream_t st) {
  KX_REQUIRE(n > 0 && n % 8 == 0, "kx_rmsnorm: n=%d must be a positive multiple of 8", n);
  KX_REQUIRE(tokens > 0, "kx_rmsnorm: tokens=%d must be positive", tokens);
  hipLaunchKernelGGL(rmsnorm_k, dim3(tokens), dim3(256), 0, st, x, w, y, n, x_stride, y_stride, eps);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

// scratch: tokens * ARGMAX_PARTS floats and as many uint32
int kx_argmax_launch(const float *logits, int tokens, int n, int stride, uint32_t *out, float *scratch, hipStream_t st) {
  float *pv = scratch;
  uint32_t *pi = (uint32_t *)(scratch + (size_t)tokens * ARGMAX_PARTS);
  hipLaunchKernelGGL(argmax_part_k, dim3(ARGMAX_PARTS, tokens), dim3(256), 0, st, logits, n, stride, pv, pi);
  KX_LAUNCH_CHECK();
  hipLaunchKernelGGL(argmax_final_k, dim3(tokens), dim3(64), 0, st, pv, pi, out);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

extern "C" int kx_rmsnorm(const void *d_x, const void *d_w, void *d_y, int32_t tokens, int32_t n, float eps,
                          void *stream) {
  KX_REQUIRE(d_x && d_w && d_y, "kx_rmsnorm: null pointer");
  return kx_rmsnorm_launch((const uint16_t *)d_x, (const uint16_t *)d_w, (uint16_t *)d_y, tokens, n, n, n, eps,
                           kx_stream(stream));
}

// sample_lm_head (:718-734) as an operator: bf16-rounded logits of the normed rows, then argmax_k's choice (:477-493)
extern "C" int kx_lm_head_argmax(const void *d_w, const void *d_n, void *d_logits, void *d_ids, int32_t vocab,
                                 int32_t hidden, int32_t tokens, void *d_scratch, void *stream) {
  KX_REQUIRE(d_w && d_n && d_logits && d_ids && d_scratch, "kx_lm_head_argmax: null pointer");
  KX_REQUIRE(vocab > 0 && tokens > 0, "kx_lm_head_argmax: vocab=%d tokens=%d must be positive", vocab, tokens);
  KxGemvArgs a = {};
  a.w0 = (const uint16_t *)d_w; a.x = (const uint16_t *)d_n; a.x_stride = hidden;
  a.out = d_logits; a.out_stride = vocab; a.rows = vocab; a.cols = hidden; a.tokens = tokens;
  int rc = kx_gemv_launch(KX_EPI_ARGMAX, a, kx_stream(stream));
  if (rc) return rc;
  return kx_argmax_launch((const float *)d_logits, tokens, vocab, vocab, (uint32_t *)d_ids, (float *)d_scratch, kx_stream(stream));
}

// ---- the same operator for callers that may not allocate ---------------------------------------
// The per-token argmax partials (ARGMAX_PARTS values and indices per token) live in a file-scope device
// array instead of a caller's buffer.  Every GPU holds its own copy of the array at its own address, so
// the address is looked up once per device, with that device current, and kept.
constexpr int KX_STATIC_ARGMAX_TOKENS = 256;
constexpr int KX_STATIC_MAX_DEVICES = 64;
static __device__ __align__(256) unsigned char g_argmax_scratch[KX_STATIC_ARGMAX_TOKENS * ARGMAX_PARTS * 8];
static std::mutex g_argmax_scratch_mu;
static void *g_argmax_scratch_ptr[KX_STATIC_MAX_DEVICES];

static int argmax_scratch_for_current_device(void **out) {
  int dev = -1;
  KX_HIP(hipGetDevice(&dev));
  KX_REQUIRE(dev >= 0 && dev < KX_STATIC_MAX_DEVICES, "kx_lm_head_argmax_static: device %d is beyond the %d this library keeps an address for",
             dev, KX_STATIC_MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_argmax_scratch_mu);
  if (!g_argmax_scratch_ptr[dev]) {
    void *p = nullptr;
    KX_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_argmax_scratch)));
    KX_REQUIRE(p != nullptr, "kx_lm_head_argmax_static: hipGetSymbolAddress gave no address on device %d", dev);
    g_argmax_scratch_ptr[dev] = p;
  }
  *out = g_argmax_scratch_ptr[dev];
  return KX_OK;
}

extern "C" int kx_static_scratch_init(void) {
  void *p = nullptr;
  return argmax_scratch_for_current_device(&p);
}

extern "C" int kx_lm_head_argmax_static(const void *d_w, const void *d_n, void *d_logits, void *d_ids, int32_t vocab,
                                        int32_t hidden, int32_t tokens, void *stream) {
  KX_REQUIRE(d_w && d_n && d_logits && d_ids, "kx_lm_head_argmax_static: null pointer");
  KX_REQUIRE(vocab > 0 && tokens > 0, "kx_lm_head_argmax_static: vocab=%d tokens=%d must be positive", vocab, tokens);
  KX_REQUIRE(tokens <= KX_STATIC_ARGMAX_TOKENS,
             "kx_lm_head_argmax_static: tokens=%d is more than the %d rows the built-in scratch holds; use kx_lm_head_argmax with a buffer of your own",
             tokens, KX_STATIC_ARGMAX_TOKENS);
  // the array is the current device's: pointers that live on another device would be handed this device's array
  int dev = -1;
  hipPointerAttribute_t attr;
  KX_HIP(hipGetDevice(&dev));
  KX_HIP(hipPointerGetAttributes(&attr, d_logits));
  KX_REQUIRE(attr.device == dev, "kx_lm_head_argmax_static: d_logits lives on device %d, the current device is %d: make the buffers' device current",
             attr.device, dev);
  void *scratch = nullptr;
  int rc = argmax_scratch_for_current_device(&scratch);
  if (rc) return rc;
  // every partial of rows [0, tokens) is written by the first argmax kernel before the second reads it: nothing to clear
  return kx_lm_head_argmax(d_w, d_n, d_logits, d_ids, vocab, hidden, tokens, scratch, stream);
}

extern "C" int kx_gemv_bf16(const void *d_w, const void *d_x, void *d_y, int32_t rows, int32_t cols,
                            int32_t tokens, int out_f32, void *stream) {
  KX_REQUIRE(d_w && d_x && d_y, "kx_gemv_bf16: null pointer");
  KxGemvArgs a = {};
  a.w0 = (const uint16_t *)d_w; a.x = (const uint16_t *)d_x; a.x_stride = cols;
  a.out = d_y; a.out_stride = rows; a.rows = rows; a.cols = cols; a.tokens = tokens;
  return kx_gemv_launch(out_f32 ? KX_EPI_F32 : KX_EPI_BF16, a, kx_stream(stream));
}
