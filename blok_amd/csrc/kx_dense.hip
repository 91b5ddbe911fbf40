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
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_math.h"

namespace {

typedef unsigned int kx_u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint4 ld_stream16(const uint16_t *p) {
  kx_u32x4 v = __builtin_nontemporal_load((const kx_u32x4 *)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float bf_lo(uint32_t u) { return kx_bits_f32(u << 16); }
__device__ __forceinline__ float bf_hi(uint32_t u) { return kx_bits_f32(u & 0xffff0000u); }

__device__ __forceinline__ float wave_sum(float v) {
  v += __shfl_xor(v, 32);
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 8);
  v += __shfl_xor(v, 4);
  v += __shfl_xor(v, 2);
  v += __shfl_xor(v, 1);
  return v;
}

__device__ __forceinline__ void unpack8(float (&f)[8], uint4 u) {
  f[0] = bf_lo(u.x); f[1] = bf_hi(u.x); f[2] = bf_lo(u.y); f[3] = bf_hi(u.y);
  f[4] = bf_lo(u.z); f[5] = bf_hi(u.z); f[6] = bf_lo(u.w); f[7] = bf_hi(u.w);
}

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
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) ws[threadIdx.x >> 6] = v;
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

// ---- GEMV -------------------------------------------------------------------------
// RI rows per wave per item, TT tokens per pass, SPW slices per wave.
template <int EPI, int RI, int TT, int SPW>
__global__ void __launch_bounds__(1024) gemv_bf16_k(KxGemvArgs a) {
  extern __shared__ float part[];  // [mats][RT][TT][S]
  constexpr int MATS = (EPI == KX_EPI_SWIGLU) ? 2 : 1;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int S = a.cols >> 9;
  const int wslot = wave % a.nw, rset = wave / a.nw;  // wave owns slices wslot*SPW .. +SPW-1
  const int RT = a.rs * RI;
  const int tiles = (a.rows + RT - 1) / RT;
  const uint16_t *wm[2] = {a.w0, a.w1};

  for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int r0 = tile * RT;
    uint4 wv[MATS][RI][SPW];
#pragma unroll
    for (int i = 0; i < RI; ++i) {
      int row = r0 + rset * RI + i;
      int row_c = row < a.rows ? row : a.rows - 1;
#pragma unroll
      for (int m = 0; m < MATS; ++m)
#pragma unroll
        for (int q = 0; q < SPW; ++q) {
          int s = wslot * SPW + q;
          int s_c = s < S ? s : S - 1;
          wv[m][i][q] = ld_stream16(wm[m] + (size_t)row_c * a.cols + (size_t)s_c * 512 + lane * 8);
        }
    }
    for (int t0 = 0; t0 < a.tokens; t0 += TT) {
      float xs[TT][SPW][8];
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        int tok = min(t0 + t, a.tokens - 1);
#pragma unroll
        for (int q = 0; q < SPW; ++q) {
          int s = wslot * SPW + q;
          int s_c = s < S ? s : S - 1;
          unpack8(xs[t][q], *(const uint4 *)(a.x + (size_t)tok * a.x_stride + (size_t)s_c * 512 + lane * 8));
        }
      }
#pragma unroll
      for (int i = 0; i < RI; ++i)
#pragma unroll
        for (int m = 0; m < MATS; ++m)
#pragma unroll
          for (int q = 0; q < SPW; ++q) {
            float wf[8];
            unpack8(wf, wv[m][i][q]);
            int s = wslot * SPW + q;
#pragma unroll
            for (int t = 0; t < TT; ++t) {
              float acc = 0.0f;
#pragma unroll
              for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(wf[e], xs[t][q][e], acc);
              acc = wave_sum(acc);
              if (lane == 0 && s < S) part[((m * RT + rset * RI + i) * TT + t) * S + s] = acc;
            }
          }
      __syncthreads();
      for (int idx = threadIdx.x; idx < RT * TT; idx += blockDim.x) {
        int rt = idx % RT, t = idx / RT;
        int row = r0 + rt, tok = t0 + t;
        if (row < a.rows && tok < a.tokens) {
          const float *p0 = part + ((0 * RT + rt) * TT + t) * S;
          float y0 = p0[0];
          for (int q = 1; q < S; ++q) y0 += p0[q];
          if (EPI == KX_EPI_BF16) {
            ((uint16_t *)a.out)[(size_t)tok * a.out_stride + row] = kx_bf16_rne(y0);
          } else if (EPI == KX_EPI_F32) {
            ((float *)a.out)[(size_t)tok * a.out_stride + row] = y0;
          } else if (EPI == KX_EPI_SWIGLU) {
            const float *p1 = part + ((1 * RT + rt) * TT + t) * S;
            float y1 = p1[0];
            for (int q = 1; q < S; ++q) y1 += p1[q];
            ((uint16_t *)a.out)[(size_t)tok * a.out_stride + row] =
                kx_bf16_rne(kx_swiglu(kx_bfround(y0), kx_bfround(y1)));
          } else if (EPI == KX_EPI_RESID) {
            // x = bf(x + bf(y))  (add_k, :248-251)
            uint16_t *xr = (uint16_t *)a.out + (size_t)tok * a.out_stride + row;
            *xr = kx_bf16_rne(kx_bf16_f32(*xr) + kx_bfround(y0));
          } else if (EPI == KX_EPI_MOE_COMBINE) {
            // down = bf(sum_slot y_slot * w_slot) in slot order (:868,:871), then
            // down = bf(down + bf(shared)) (:684), then x = bf(x + down) (:877)
            float acc = 0.0f;
            for (int k = 0; k < a.topk; ++k)
              acc = __builtin_fmaf(kx_bf16_f32(a.expert_out[((size_t)tok * a.topk + k) * a.rows + row]),
                                   a.route_w[(size_t)tok * a.topk + k], acc);
            float down = kx_bfround(kx_bfround(acc) + kx_bfround(y0));
            uint16_t *xr = (uint16_t *)a.out + (size_t)tok * a.out_stride + row;
            if (a.flags & 1u) *xr = kx_bf16_rne(down);
            else *xr = kx_bf16_rne(kx_bf16_f32(*xr) + down);
          } else if (EPI == KX_EPI_ARGMAX) {
            // bf16-rounded logits; the per-tile argmax is reduced by a second kernel
            ((float *)a.out)[(size_t)tok * a.out_stride + row] = kx_bfround(y0);
          }
        }
      }
      __syncthreads();
    }
  }
}

// lowest-index argmax over bf16-rounded logits (sample_lm_head :718-734, argmax_k :477-493)
__global__ void __launch_bounds__(1024) argmax_rows_k(const float *__restrict__ logits, int n, int stride,
                                                      uint32_t *__restrict__ out) {
  __shared__ float sv[16];
  __shared__ uint32_t si[16];
  const float *p = logits + (size_t)blockIdx.x * stride;
  float best = -__builtin_inff();
  uint32_t bi = 0;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = p[i];
    if (v > best) { best = v; bi = (uint32_t)i; }
  }
  for (int m = 32; m; m >>= 1) {
    float ov = __shfl_xor(best, m);
    uint32_t oi = (uint32_t)__shfl_xor((int)bi, m);
    if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
  }
  if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w)
      if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
    out[blockIdx.x] = bi;
  }
}

template <int EPI, int RI, int TT>
void launch_spw(const KxGemvArgs &a, int spw, dim3 g, dim3 b, size_t lds, hipStream_t st) {
  if (spw == 1) hipLaunchKernelGGL((gemv_bf16_k<EPI, RI, TT, 1>), g, b, lds, st, a);
  else if (spw == 2) hipLaunchKernelGGL((gemv_bf16_k<EPI, RI, TT, 2>), g, b, lds, st, a);
  else hipLaunchKernelGGL((gemv_bf16_k<EPI, RI, TT, 3>), g, b, lds, st, a);
}

template <int EPI>
void launch_tt(const KxGemvArgs &a, int tt, int spw, dim3 g, dim3 b, size_t lds, hipStream_t st) {
  if (tt == 1) launch_spw<EPI, KX_GEMV_RI, 1>(a, spw, g, b, lds, st);
  else if (tt == 2) launch_spw<EPI, KX_GEMV_RI, 2>(a, spw, g, b, lds, st);
  else launch_spw<EPI, KX_GEMV_RI, 4>(a, spw, g, b, lds, st);
}

}  // namespace

int kx_gemv_launch(int epi, KxGemvArgs a, hipStream_t st) {
  KX_REQUIRE(a.cols > 0 && a.cols % 512 == 0, "kx_gemv: cols=%d must be a positive multiple of 512", a.cols);
  KX_REQUIRE(a.rows > 0 && a.tokens > 0, "kx_gemv: rows=%d tokens=%d must be positive", a.rows, a.tokens);
  const int S = a.cols / 512;
  const int spw = (S + 15) / 16;
  KX_REQUIRE(spw <= 3, "kx_gemv: cols=%d exceeds 24576", a.cols);
  a.nw = (S + spw - 1) / spw;
  a.rs = a.nw >= 8 ? 1 : 8 / a.nw;
  const int tt = a.tokens >= 4 ? 4 : a.tokens >= 2 ? 2 : 1;
  const int mats = epi == KX_EPI_SWIGLU ? 2 : 1;
  const int RT = a.rs * KX_GEMV_RI;
  const size_t lds = (size_t)mats * RT * tt * S * sizeof(float);
  const int tiles = kx_cdiv(a.rows, RT);
  dim3 g(tiles < 2048 ? tiles : 2048), b(a.nw * a.rs * 64);
  switch (epi) {
    case KX_EPI_BF16: launch_tt<KX_EPI_BF16>(a, tt, spw, g, b, lds, st); break;
    case KX_EPI_F32: launch_tt<KX_EPI_F32>(a, tt, spw, g, b, lds, st); break;
    case KX_EPI_SWIGLU: launch_tt<KX_EPI_SWIGLU>(a, tt, spw, g, b, lds, st); break;
    case KX_EPI_RESID: launch_tt<KX_EPI_RESID>(a, tt, spw, g, b, lds, st); break;
    case KX_EPI_MOE_COMBINE: launch_tt<KX_EPI_MOE_COMBINE>(a, tt, spw, g, b, lds, st); break;
    case KX_EPI_ARGMAX: launch_tt<KX_EPI_ARGMAX>(a, tt, spw, g, b, lds, st); break;
    default: kx_set_error("kx_gemv: unknown epilogue %d", epi); return KX_ERR_ARG;
  }
  KX_LAUNCH_CHECK();
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

int kx_argmax_launch(const float *logits, int tokens, int n, int stride, uint32_t *out, hipStream_t st) {
  hipLaunchKernelGGL(argmax_rows_k, dim3(tokens), dim3(1024), 0, st, logits, n, stride, out);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

extern "C" int kx_rmsnorm(const void *d_x, const void *d_w, void *d_y, int32_t tokens, int32_t n, float eps,
                          void *stream) {
  KX_REQUIRE(d_x && d_w && d_y, "kx_rmsnorm: null pointer");
  return kx_rmsnorm_launch((const uint16_t *)d_x, (const uint16_t *)d_w, (uint16_t *)d_y, tokens, n, n, n, eps,
                           kx_stream(stream));
}

extern "C" int kx_gemv_bf16(const void *d_w, const void *d_x, void *d_y, int32_t rows, int32_t cols,
                            int32_t tokens, int out_f32, void *stream) {
  KX_REQUIRE(d_w && d_x && d_y, "kx_gemv_bf16: null pointer");
  KxGemvArgs a = {};
  a.w0 = (const uint16_t *)d_w; a.x = (const uint16_t *)d_x; a.x_stride = cols;
  a.out = d_y; a.out_stride = rows; a.rows = rows; a.cols = cols; a.tokens = tokens;
  return kx_gemv_launch(out_f32 ? KX_EPI_F32 : KX_EPI_BF16, a, kx_stream(stream));
}
