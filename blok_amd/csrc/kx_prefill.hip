// kx_prefill.hip -- W4A16 grouped GEMM for prefill chunks through one MoE layer.
//
// The reference has no batched prefill: it runs one decode step per prompt token
// (src/kimi_exec.cu:886) and, inside it, the per-expert loops at :845-870.  For a
// chunk of T tokens this file computes the same per-token quantities -- gate/up
// projections with SwiGLU (:853-862), down projection (:863-869), the routed
// combine (:868,:871), the shared expert (:872-875) and the residual add (:877) --
// with the tokens of each expert gathered into one GEMM.
//
// The only place MFMA is used.  Per workgroup: one expert, 128 weight rows, the
// expert's tokens in tiles of 64.  Per K step of 64 columns the packed INT4 words
// are unpacked and dequantized exactly as the reference does, w = bf((n-8)*scale)
// (:311-312), into an LDS tile of bf16; the gathered activation rows go into a
// second LDS tile; four waves each run v_mfma_f32_32x32x16_bf16 on a 64x32 slab of
// the output with fp32 accumulators.  The bf16 shared expert uses the same kernel
// with a plain copy in place of the dequant.
//
// MFMA's internal summation order is not documented, so this path is held to the
// max-rel 1e-2 bar and is never used for the token-identity runs.
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_math.h"

namespace {

typedef __bf16 kx_bf16x8 __attribute__((ext_vector_type(8)));
typedef float kx_f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 64, BN = 128, BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // bf16 elements per LDS row: 144 B keeps 16-byte reads of a column of rows spread over banks

struct PfArgs {
  const void *w0, *w1;          // INT4: packed i32 [E][N][K/8]; BF16: bf16 [E][N][K]
  const uint16_t *s0, *s1;      // INT4: bf16 scales [E][N][K/32]
  const uint16_t *x;            // bf16 activation rows of K
  uint16_t *out;                // bf16 [pairs][N]
  const int4 *work;             // {expert, first, last, _} per expert with work; nullptr: one group of n_pairs rows
  const int *pairs;             // pair ids sorted by expert; nullptr: identity
  int n_pairs, N, K, x_div;     // activation row = pair / x_div
  size_t expert_w, expert_s;    // elements between experts (words or bf16; scales)
};

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return (uint32_t)kx_bf16_rne(lo) | ((uint32_t)kx_bf16_rne(hi) << 16);
}

// dequantize one group (4 packed words, 32 weights) to 32 bf16 = 4 uint4, columns ascending
__device__ __forceinline__ void dequant_group(const uint4 v, float sc, uint4 (&o)[4]) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  const float m8 = -8.0f * sc;  // exact
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    float f[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = __builtin_fmaf((float)((w[p] >> (4 * j)) & 0xfu), sc, m8);  // == (n-8)*sc exactly
    o[p] = make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
  }
}

template <bool DUAL, bool I4>
__global__ void __launch_bounds__(256) grouped_gemm_k(PfArgs a) {
  constexpr int MATS = DUAL ? 2 : 1;
  __shared__ __attribute__((aligned(16))) uint16_t xs[BM * LDS_STRIDE];
  __shared__ __attribute__((aligned(16))) uint16_t ws[MATS][BN * LDS_STRIDE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * BN;
  int4 wk = a.work ? a.work[blockIdx.y] : make_int4(0, 0, a.n_pairs, 0);
  const int e = __builtin_amdgcn_readfirstlane(wk.x);
  if (e < 0) return;
  const int p_begin = __builtin_amdgcn_readfirstlane(wk.y), p_end = __builtin_amdgcn_readfirstlane(wk.z);
  const void *wbase[2] = {a.w0, a.w1};
  const uint16_t *sbase[2] = {a.s0, a.s1};
  // staging roles
  const int xr = tid >> 2, xc = (tid & 3) * 16;   // activation tile: row, first of 16 columns
  const int wr = tid >> 1, wg = tid & 1;          // weight tile: row, group (32 columns) of the K step

  // token tiles of the expert are spread over blockIdx.z
  for (int m0 = p_begin + blockIdx.z * BM; m0 < p_end; m0 += gridDim.z * BM) {
    kx_f32x16 acc[MATS][2];
#pragma unroll
    for (int m = 0; m < MATS; ++m)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[m][t][i] = 0.0f;
    const int pi = m0 + xr;
    const bool x_valid = pi < p_end;
    const int pair = x_valid ? (a.pairs ? a.pairs[pi] : pi) : 0;
    const uint16_t *xrow = a.x + (size_t)(pair / a.x_div) * a.K + xc;
    const int wrow = min(n0 + wr, a.N - 1);
    for (int k0 = 0; k0 < a.K; k0 += BK) {
      // global loads of this K step
      uint4 xv0 = make_uint4(0, 0, 0, 0), xv1 = xv0;
      if (x_valid) { xv0 = *(const uint4 *)(xrow + k0); xv1 = *(const uint4 *)(xrow + k0 + 8); }
      uint4 wq[MATS][4];
#pragma unroll
      for (int m = 0; m < MATS; ++m) {
        if (I4) {
          const uint32_t *pw = (const uint32_t *)wbase[m] + (size_t)e * a.expert_w + (size_t)wrow * (a.K >> 3) + ((k0 >> 3) + wg * 4);
          const float sc = kx_bf16_f32(sbase[m][(size_t)e * a.expert_s + (size_t)wrow * (a.K >> 5) + (k0 >> 5) + wg]);
          dequant_group(*(const uint4 *)pw, sc, wq[m]);
        } else {
          const uint16_t *pw = (const uint16_t *)wbase[m] + (size_t)e * a.expert_w + (size_t)wrow * a.K + k0 + wg * 32;
#pragma unroll
          for (int p = 0; p < 4; ++p) wq[m][p] = ((const uint4 *)pw)[p];
        }
      }
      __syncthreads();  // the previous K step's fragments have been read
      *(uint4 *)(xs + xr * LDS_STRIDE + xc) = xv0;
      *(uint4 *)(xs + xr * LDS_STRIDE + xc + 8) = xv1;
#pragma unroll
      for (int m = 0; m < MATS; ++m)
#pragma unroll
        for (int p = 0; p < 4; ++p) *(uint4 *)(ws[m] + wr * LDS_STRIDE + wg * 32 + p * 8) = wq[m][p];
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < BK; kk += 16) {
        // operand layout of v_mfma_f32_32x32x16_bf16: lane l holds row (l % 32), k = 8*(l / 32) .. +7
        const int kcol = kk + (lane >> 5) * 8;
        const kx_bf16x8 a0 = *(const kx_bf16x8 *)(xs + (lane & 31) * LDS_STRIDE + kcol);
        const kx_bf16x8 a1 = *(const kx_bf16x8 *)(xs + (32 + (lane & 31)) * LDS_STRIDE + kcol);
#pragma unroll
        for (int m = 0; m < MATS; ++m) {
          const kx_bf16x8 b = *(const kx_bf16x8 *)(ws[m] + (wave * 32 + (lane & 31)) * LDS_STRIDE + kcol);
          acc[m][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b, acc[m][0], 0, 0, 0);
          acc[m][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b, acc[m][1], 0, 0, 0);
        }
      }
    }
    // epilogue: D[i][j], j = lane % 32 (weight row), i = 8*(v/4) + 4*(lane/32) + v%4 (token of the tile)
    const int n = n0 + wave * 32 + (lane & 31);
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int i = t * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        const int po = m0 + i;
        if (po < p_end && n < a.N) {
          const int pr = a.pairs ? a.pairs[po] : po;
          float r = acc[0][t][v];
          if (DUAL) r = kx_swiglu(kx_bfround(r), kx_bfround(acc[1][t][v]));
          a.out[(size_t)pr * a.N + n] = kx_bf16_rne(r);
        }
      }
    __syncthreads();
  }
}

// x[t][r] = bf(x + bf(bf(sum_slot eout[t*topk+slot][r] * w[t][slot]) + sy[t][r]))  (:868-877)
__global__ void __launch_bounds__(256) moe_combine_k(const uint16_t *__restrict__ eout, const float *__restrict__ rw,
                                                     const uint16_t *__restrict__ sy, uint16_t *__restrict__ x, int hidden,
                                                     int topk, uint32_t flags) {
  const int t = blockIdx.y, r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= hidden) return;
  float acc = 0.0f;
  for (int k = 0; k < topk; ++k)
    acc = __builtin_fmaf(kx_bf16_f32(eout[((size_t)t * topk + k) * hidden + r]), rw[(size_t)t * topk + k], acc);
  const float down = kx_bfround(kx_bfround(acc) + kx_bf16_f32(sy[(size_t)t * hidden + r]));
  uint16_t *xr = x + (size_t)t * hidden + r;
  *xr = (flags & 1u) ? kx_bf16_rne(down) : kx_bf16_rne(kx_bf16_f32(*xr) + down);
}

}  // namespace

int kx_grouped_gemm_launch(bool dual, bool i4, const void *w0, const uint16_t *s0, const void *w1, const uint16_t *s1,
                           const uint16_t *x, uint16_t *out, const int4 *work, const int *pairs, int n_pairs, int n_slots,
                           int N, int K, int x_div, size_t expert_w, size_t expert_s, int n_pairs_max, hipStream_t st) {
  KX_REQUIRE(K > 0 && K % 64 == 0, "kx_grouped_gemm: K=%d must be a positive multiple of 64", K);
  KX_REQUIRE(N > 0, "kx_grouped_gemm: N=%d must be positive", N);
  PfArgs a;
  a.w0 = w0; a.w1 = w1; a.s0 = s0; a.s1 = s1; a.x = x; a.out = out; a.work = work; a.pairs = pairs;
  a.n_pairs = n_pairs; a.N = N; a.K = K; a.x_div = x_div; a.expert_w = expert_w; a.expert_s = expert_s;
  const int max_rows = work ? n_pairs_max : n_pairs;
  int mz = kx_cdiv(max_rows, BM);
  mz = mz < 1 ? 1 : mz > 64 ? 64 : mz;
  dim3 g(kx_cdiv(N, BN), work ? n_slots : 1, mz), b(256);
  if (dual && i4) hipLaunchKernelGGL((grouped_gemm_k<true, true>), g, b, 0, st, a);
  else if (dual) hipLaunchKernelGGL((grouped_gemm_k<true, false>), g, b, 0, st, a);
  else if (i4) hipLaunchKernelGGL((grouped_gemm_k<false, true>), g, b, 0, st, a);
  else hipLaunchKernelGGL((grouped_gemm_k<false, false>), g, b, 0, st, a);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

int kx_moe_combine_launch(const uint16_t *eout, const float *rw, const uint16_t *sy, uint16_t *x, int tokens, int hidden,
                          int topk, uint32_t flags, hipStream_t st) {
  hipLaunchKernelGGL(moe_combine_k, dim3(kx_cdiv(hidden, 256), tokens), dim3(256), 0, st, eout, rw, sy, x, hidden, topk, flags);
  KX_LAUNCH_CHECK();
  return KX_OK;
}
