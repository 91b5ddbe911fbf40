// kx_prefill.hip -- W4A16 grouped GEMM for prefill chunks through one MoE layer.
//
// The reference has no batched prefill: it runs one decode step per prompt token
// (src/kimi_exec.cu:886) and, inside it, the per-expert loops at :845-870.  For a
// chunk of T tokens this file computes the same per-token quantities -- gate/up
// projections with SwiGLU (:853-862), down projection (:863-869), the routed
// combine (:868,:871), the shared expert (:872-875) and the residual add (:877) --
// with the tokens of each expert gathered into one GEMM.
//
// The only place MFMA is used.  Per workgroup (4 waves): one expert, 128 weight rows, the
// expert's tokens in tiles of 128.  Wave w owns weight rows 32 w .. +31 for all 128 tokens
// (fp32 accumulators of v_mfma_f32_32x32x16_bf16).  Per K step of 64 columns:
//  * weights never touch LDS: lane (r, h) = (lane % 32, lane / 32) loads the 16 bytes of row r
//    that hold columns 32 h .. +31 of the step -- one quantization group, four packed words --
//    and dequantizes word j to the reference's values, w = bf((n-8)*scale) (:311-312), which
//    is exactly the B operand of the step's j-th MFMA when that MFMA contracts over columns
//    {8 j .. +7} and {32 + 8 j .. +7} (the contraction order within a step is free, the
//    activation operand uses the same columns);
//  * the gathered activation rows go through a double-buffered LDS tile, one barrier per step;
//  * the global loads of step k+1 are in flight while step k is computed.
// The bf16 shared expert and the router gate use the same kernel with plain loads in place
// of the dequant.
//
// Dequant without integer conversion: (w & 0x000F000F) | 0x64006400 is the f16 pair
// (1024+n0, 1024+n4), (w & 0x00F000F0) | 0x64006400 is (1024+16 n1, 1024+16 n5), w >> 8 gives
// n2,n6,n3,n7 the same way; fma(f16, s, -1032 s) = (n-8) s and fma(f16, s/16, -72 s) = (n-8) s
// are exact in fp32 (4-bit times 8-bit significands), and one v_cvt_pk_bf16_f32 rounds two of
// them to nearest-even.
//
// MFMA's internal summation order is not documented, so this path is held to the
// max-rel 1e-2 bar and is never used for the token-identity runs.
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_math.h"

#include <type_traits>

namespace {

typedef __bf16 kx_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 kx_bf16x2 __attribute__((ext_vector_type(2)));
typedef float kx_f32x2 __attribute__((ext_vector_type(2)));
typedef float kx_f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 kx_h2 __attribute__((ext_vector_type(2)));

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // bf16 elements per LDS row: 144 B keeps 16-byte reads of a column of rows spread over banks
constexpr int PF_THREADS = 256;

struct PfArgs {
  const void *w0, *w1;          // INT4: packed i32 [E][N][K/8]; BF16: bf16 [E][N][K]
  const uint16_t *s0, *s1;      // INT4: bf16 scales [E][N][K/32]
  const uint16_t *x;            // bf16 activation rows of K
  void *out;                    // bf16 [pairs][N], or f32 when out_f32
  const int4 *work;             // {expert, first, last, _} per expert with work; nullptr: one group of n_pairs rows
  const int *pairs;             // pair ids sorted by expert; nullptr: identity
  int n_pairs, N, K, x_div;     // activation row = pair / x_div
  size_t expert_w, expert_s;    // elements between experts (words or bf16; scales)
  int out_f32;                  // single matrix only: store the fp32 accumulators unrounded
};

__device__ __forceinline__ uint32_t pf_and_or(uint32_t a, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(magic));
  return r;
}
__device__ __forceinline__ uint32_t pf_pack(float lo, float hi) {
  kx_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, kx_bf16x2));
}

// dequantize one packed word (8 weights) to 8 bf16, columns ascending
__device__ __forceinline__ kx_bf16x8 dequant_word(uint32_t w, float sc, float sc16, float c0, float c1, uint32_t magic) {
  const uint32_t w8 = w >> 8;
  const kx_h2 a = __builtin_bit_cast(kx_h2, pf_and_or(w, 0x000F000Fu, magic));   // n0, n4
  const kx_h2 b = __builtin_bit_cast(kx_h2, pf_and_or(w, 0x00F000F0u, magic));   // 16 n1, 16 n5
  const kx_h2 c = __builtin_bit_cast(kx_h2, pf_and_or(w8, 0x000F000Fu, magic));  // n2, n6
  const kx_h2 d = __builtin_bit_cast(kx_h2, pf_and_or(w8, 0x00F000F0u, magic));  // 16 n3, 16 n7
  const float f0 = __builtin_fmaf((float)a.x, sc, c0), f4 = __builtin_fmaf((float)a.y, sc, c0);
  const float f1 = __builtin_fmaf((float)b.x, sc16, c1), f5 = __builtin_fmaf((float)b.y, sc16, c1);
  const float f2 = __builtin_fmaf((float)c.x, sc, c0), f6 = __builtin_fmaf((float)c.y, sc, c0);
  const float f3 = __builtin_fmaf((float)d.x, sc16, c1), f7 = __builtin_fmaf((float)d.y, sc16, c1);
  return __builtin_bit_cast(kx_bf16x8, make_uint4(pf_pack(f0, f1), pf_pack(f2, f3), pf_pack(f4, f5), pf_pack(f6, f7)));
}

template <bool DUAL, bool I4>
__global__ void __launch_bounds__(PF_THREADS, 2) grouped_gemm_k(PfArgs a) {
  constexpr int MATS = DUAL ? 2 : 1;
  constexpr int XT = BM * LDS_STRIDE;  // elements of one activation tile
  __shared__ __attribute__((aligned(16))) uint16_t xs_lds[2 * XT];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 31, lh = lane >> 5;
  const int n0 = blockIdx.x * BN;
  int4 wk = a.work ? a.work[blockIdx.y] : make_int4(0, 0, a.n_pairs, 0);
  const int e = __builtin_amdgcn_readfirstlane(wk.x);
  if (e < 0) return;
  const int p_begin = __builtin_amdgcn_readfirstlane(wk.y), p_end = __builtin_amdgcn_readfirstlane(wk.z);
  uint32_t magic;
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));
  const int nk = a.K / BK;
  // this lane's weight row and its 32-column half of every K step
  const int wrow = min(n0 + wave * 32 + lr, a.N - 1);
  const uint32_t *wq_ptr[MATS];
  const uint16_t *wb_ptr[MATS], *sc_ptr[MATS];
#pragma unroll
  for (int m = 0; m < MATS; ++m) {
    const void *wbase = m ? a.w1 : a.w0;
    wq_ptr[m] = (const uint32_t *)wbase + (size_t)e * a.expert_w + (size_t)wrow * (a.K >> 3) + lh * 4;
    wb_ptr[m] = (const uint16_t *)wbase + (size_t)e * a.expert_w + (size_t)wrow * a.K + lh * 32;
    sc_ptr[m] = (m ? a.s1 : a.s0) + (I4 ? (size_t)e * a.expert_s + (size_t)wrow * (a.K >> 5) + lh : 0);
  }
  // activation staging: thread -> rows tid/4 and 64 + tid/4, 16 columns from (tid%4)*16
  const int xr = tid >> 2, xc = (tid & 3) * 16;

  for (int m0 = p_begin + blockIdx.z * BM; m0 < p_end; m0 += gridDim.z * BM) {
    const int nb = min(4, (p_end - m0 + 31) >> 5);  // 32-token blocks that hold tokens
    const uint16_t *xrow[2];
    bool x_valid[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int pi = m0 + q * 64 + xr;
      x_valid[q] = pi < p_end;
      const int pair = x_valid[q] ? (a.pairs ? a.pairs[pi] : pi) : 0;
      xrow[q] = a.x + (size_t)(pair / a.x_div) * a.K + xc;
    }

    // the tile with NB token blocks, NB a compile-time constant so that the K loop has no branches
    auto run = [&](auto nb_c) {
      constexpr int NB = decltype(nb_c)::value;
      constexpr int XQ = NB > 2 ? 2 : 1;  // halves of the activation tile that are staged
      kx_f32x16 acc[MATS][NB];
#pragma unroll
      for (int m = 0; m < MATS; ++m)
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[m][t][i] = 0.0f;
      struct WRaw {
        uint4 q[MATS];      // INT4: the group's four packed words
        float sc[MATS];
        uint4 b[MATS][I4 ? 1 : 4];  // BF16: 32 columns
      };
      uint4 xv[XQ][2];
      auto load_w = [&](WRaw &r, int ks) {
#pragma unroll
        for (int m = 0; m < MATS; ++m) {
          if (I4) {
            r.q[m] = *(const uint4 *)(wq_ptr[m] + ks * 8);
            r.sc[m] = kx_bf16_f32(sc_ptr[m][ks * 2]);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) r.b[m][j] = *(const uint4 *)(wb_ptr[m] + ks * BK + j * 8);
          }
        }
      };
      auto load_x = [&](int ks) {
#pragma unroll
        for (int q = 0; q < XQ; ++q) {
          xv[q][0] = xv[q][1] = make_uint4(0, 0, 0, 0);
          if (x_valid[q]) { xv[q][0] = *(const uint4 *)(xrow[q] + ks * BK); xv[q][1] = *(const uint4 *)(xrow[q] + ks * BK + 8); }
        }
      };
      auto store_x = [&](uint16_t *st) {
#pragma unroll
        for (int q = 0; q < XQ; ++q) {
          *(uint4 *)(st + (q * 64 + xr) * LDS_STRIDE + xc) = xv[q][0];
          *(uint4 *)(st + (q * 64 + xr) * LDS_STRIDE + xc + 8) = xv[q][1];
        }
      };
      // one K step on the weights in r; the activations of step ks are in LDS tile ks % 2.
      // MFMA j of the step contracts over columns 8 j .. +7 (lanes 0-31) and 32 + 8 j .. +7 (lanes 32-63).
      // Software pipeline: the operands of MFMA group j+1 (LDS reads of the activations, dequant of the
      // weights) are produced while the matrix cores run group j.
      auto dequant_j = [&](const WRaw &r, int j, kx_bf16x8 (&b)[MATS]) {
#pragma unroll
        for (int m = 0; m < MATS; ++m) {
          if (I4) {
            const float sc = r.sc[m];
            const uint32_t w = j == 0 ? r.q[m].x : j == 1 ? r.q[m].y : j == 2 ? r.q[m].z : r.q[m].w;
            b[m] = dequant_word(w, sc, sc * 0.0625f, -1032.0f * sc, -72.0f * sc, magic);
          } else {
            b[m] = __builtin_bit_cast(kx_bf16x8, r.b[m][j]);
          }
        }
      };
      auto read_a = [&](const uint16_t *xs, int j, kx_bf16x8 (&av)[NB]) {
        const int kcol = lh * 32 + j * 8;
#pragma unroll
        for (int t = 0; t < NB; ++t) av[t] = *(const kx_bf16x8 *)(xs + (t * 32 + lr) * LDS_STRIDE + kcol);
      };
      constexpr int VPER = I4 ? (34 * MATS + NB * MATS - 1) / (NB * MATS) : 0;  // VALU instructions per MFMA
      auto mfma_group = [&](const kx_bf16x8 (&av)[NB], const kx_bf16x8 (&b)[MATS], auto with_valu) {
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
          for (int m = 0; m < MATS; ++m) acc[m][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[t], b[m], acc[m][t], 0, 0, 0);
        // scheduling: one MFMA, then a share of the VALU work that prepares the next group
#pragma unroll
        for (int i = 0; i < NB * MATS; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if constexpr (decltype(with_valu)::value) __builtin_amdgcn_sched_group_barrier(0x002, VPER, 0);
        }
      };
      auto step = [&](const WRaw &r, int ks) {
        const uint16_t *xs = xs_lds + (ks & 1) * XT;
        kx_bf16x8 b0[MATS], b1[MATS], a0[NB], a1[NB];
        dequant_j(r, 0, b0);
        read_a(xs, 0, a0);
        read_a(xs, 1, a1);
        dequant_j(r, 1, b1);
        mfma_group(a0, b0, std::true_type{});
        read_a(xs, 2, a0);
        dequant_j(r, 2, b0);
        mfma_group(a1, b1, std::true_type{});
        read_a(xs, 3, a1);
        dequant_j(r, 3, b1);
        mfma_group(a0, b0, std::true_type{});
        mfma_group(a1, b1, std::false_type{});
      };

      // weights and activations are fetched one K step ahead (registers; two LDS tiles)
      WRaw w0, w1;
      load_w(w0, 0);
      load_x(0);
      store_x(xs_lds);
      __syncthreads();
      for (int ks = 0; ks < nk; ks += 2) {
        if (ks + 1 < nk) { load_w(w1, ks + 1); load_x(ks + 1); }
        step(w0, ks);
        if (ks + 1 < nk) store_x(xs_lds + XT);
        __syncthreads();
        if (ks + 1 < nk) {
          if (ks + 2 < nk) { load_w(w0, ks + 2); load_x(ks + 2); }
          step(w1, ks + 1);
          if (ks + 2 < nk) store_x(xs_lds);
          __syncthreads();
        }
      }
      // epilogue: D[i][j], j = lane % 32 (weight row), i = 8*(v/4) + 4*(lane/32) + v%4 (token of the 32-token block)
      const int n = n0 + wave * 32 + lr;
      if (n < a.N) {
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int po = m0 + t * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
            if (po < p_end) {
              const int pr = a.pairs ? a.pairs[po] : po;
              float r = acc[0][t][v];
              if (DUAL) r = kx_swiglu(kx_bfround(r), kx_bfround(acc[1][t][v]));
              if (!DUAL && a.out_f32) ((float *)a.out)[(size_t)pr * a.N + n] = r;
              else ((uint16_t *)a.out)[(size_t)pr * a.N + n] = kx_bf16_rne(r);
            }
          }
      }
      __syncthreads();  // the next token tile starts by overwriting LDS tile 0
    };
    if (nb == 1) run(std::integral_constant<int, 1>{});
    else if (nb == 2) run(std::integral_constant<int, 2>{});
    else if (nb == 3) run(std::integral_constant<int, 3>{});
    else run(std::integral_constant<int, 4>{});
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
                           const uint16_t *x, void *out, bool out_f32, const int4 *work, const int *pairs, int n_pairs,
                           int n_slots, int N, int K, int x_div, size_t expert_w, size_t expert_s, int n_pairs_max,
                           hipStream_t st) {
  KX_REQUIRE(K > 0 && K % 64 == 0, "kx_grouped_gemm: K=%d must be a positive multiple of 64", K);
  KX_REQUIRE(N > 0, "kx_grouped_gemm: N=%d must be positive", N);
  KX_REQUIRE(!(dual && out_f32), "kx_grouped_gemm: fp32 output is for a single matrix");
  PfArgs a;
  a.w0 = w0; a.w1 = w1; a.s0 = s0; a.s1 = s1; a.x = x; a.out = out; a.work = work; a.pairs = pairs;
  a.n_pairs = n_pairs; a.N = N; a.K = K; a.x_div = x_div; a.expert_w = expert_w; a.expert_s = expert_s;
  a.out_f32 = out_f32 ? 1 : 0;
  const int max_rows = work ? n_pairs_max : n_pairs;
  int mz = kx_cdiv(max_rows, BM);
  mz = mz < 1 ? 1 : mz > 64 ? 64 : mz;
  dim3 g(kx_cdiv(N, BN), work ? n_slots : 1, mz), b(PF_THREADS);
  const size_t lds = 0;
  if (dual && i4) hipLaunchKernelGGL((grouped_gemm_k<true, true>), g, b, lds, st, a);
  else if (dual) hipLaunchKernelGGL((grouped_gemm_k<true, false>), g, b, lds, st, a);
  else if (i4) hipLaunchKernelGGL((grouped_gemm_k<false, true>), g, b, lds, st, a);
  else hipLaunchKernelGGL((grouped_gemm_k<false, false>), g, b, lds, st, a);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

int kx_moe_combine_launch(const uint16_t *eout, const float *rw, const uint16_t *sy, uint16_t *x, int tokens, int hidden,
                          int topk, uint32_t flags, hipStream_t st) {
  hipLaunchKernelGGL(moe_combine_k, dim3(kx_cdiv(hidden, 256), tokens), dim3(256), 0, st, eout, rw, sy, x, hidden, topk, flags);
  KX_LAUNCH_CHECK();
  return KX_OK;
}
