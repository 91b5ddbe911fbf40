// kx_skinny.hip -- dense projections for decode batches of 16 to 32 sequences: y[t, r] = sum_k x[t, k] w[r, k] with
// bf16 weights [rows, cols] streamed once and the tokens as the other side of a matrix-core product.
//
// Reference: matvec_bf16_k / matvec_bf16_f32_k (src/kimi_exec.cu:272-298) called once per token; the epilogues are
// add_k (:248-251), silu_mul_k (:253-256) and the bf16 rounding of the logits (:718-734).
//
// A GEMV kernel is bound by its fma count from about 16 tokens on (every weight meets every token on the VALU), and
// the grouped prefill GEMM of kx_prefill.hip, built for 128-token tiles of many experts, leaves most of the chip idle
// on one 32-token tile.  Here a workgroup of 8 waves owns 32 weight rows and walks the columns in steps of 512; in step
// j wave w takes columns 512 j + 64 w .. + 63, so that the eight waves read 1 KB of every row together (a wave on its
// own would touch 128 bytes of 32 rows, a new DRAM page with every access).  Load m of a step takes, for lane
// (r, h) = (lane % 32, lane / 32), the 16 bytes of row r at columns 512 j + 64 w + 16 m + 8 h, and the same bytes of
// token r's activations (from L2: the activations are small and shared by every workgroup).  Load m feeds
// v_mfma_f32_32x32x16_bf16 number m: its 16 contraction indices are those 16 columns, the same for both operands.  Two steps are in flight while one is multiplied.  The eight partial
// 32 x 32 tiles are summed through LDS in wave order and the epilogue runs on the sum.
// Sums are fp32 over exact bf16 products in another order than the GEMV's: this path is held to the 1e-2 bar, like the
// other matrix-core paths, and serves batches the token-identity checks do not run on.
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_math.h"

namespace {

typedef __bf16 kx_bf16x8 __attribute__((ext_vector_type(8)));
typedef float kx_f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int kx_u32x4 __attribute__((ext_vector_type(4)));

struct SkinnyArgs {
  const uint16_t *w0, *w1;  // bf16 [rows, cols]; w1 for the two-matrix SwiGLU form
  const uint16_t *x;        // bf16 [tokens, x_stride]
  void *out;                // [tokens, out_stride]: bf16, or f32 (see mode)
  int rows, cols, tokens, x_stride, out_stride, mode;
};

__device__ __forceinline__ kx_u32x4 ld_w(const uint16_t *p) { return __builtin_nontemporal_load((const kx_u32x4 *)p); }

// NW waves per workgroup
template <bool DUAL, int NW>
__global__ void __launch_bounds__(NW * 64) skinny_gemm_k(SkinnyArgs a) {
  constexpr int MATS = DUAL ? 2 : 1;
  __shared__ float part[MATS][NW][32][32];  // [matrix][wave][token][row]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int row0 = blockIdx.x * 32;
  const int steps = a.cols / (NW * 64);  // steps of NW * 64 columns (the host checks that they divide cols)
  const int wrow = min(row0 + r, a.rows - 1), tok = min(r, a.tokens - 1);
  const uint16_t *wp[MATS];
  wp[0] = a.w0 + (size_t)wrow * a.cols + wave * 64 + 8 * h;
  if (DUAL) wp[MATS - 1] = a.w1 + (size_t)wrow * a.cols + wave * 64 + 8 * h;
  const uint16_t *xp = a.x + (size_t)tok * a.x_stride + wave * 64 + 8 * h;
  kx_f32x16 acc[MATS];
#pragma unroll
  for (int m = 0; m < MATS; ++m)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[m][v] = 0.0f;

  struct Step { kx_u32x4 w[MATS][4], x[4]; };
  auto load = [&](Step &s, int j) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int m = 0; m < MATS; ++m) s.w[m][q] = ld_w(wp[m] + j * (NW * 64) + q * 16);
      s.x[q] = *(const kx_u32x4 *)(xp + j * (NW * 64) + q * 16);
    }
  };
  auto mul = [&](const Step &s) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int m = 0; m < MATS; ++m)
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(kx_bf16x8, s.x[q]), __builtin_bit_cast(kx_bf16x8, s.w[m][q]),
                                                         acc[m], 0, 0, 0);
  };
  // Three buffers: two steps in flight while one is multiplied.  Every load is unconditional (past the end the last
  // step is requested again and never used), so that the waits in front of the products count exactly the loads
  // behind them: after a load under a condition the compiler would wait for everything in flight.
  // The scheduler is kept from moving a step's loads behind the products in front of them (it would, to save
  // registers, and the kernel would wait for every step it is about to multiply).
  const int last = steps - 1;
  Step s0, s1, s2;
  load(s0, 0);
  load(s1, min(1, last));
  __builtin_amdgcn_sched_barrier(0);
  for (int j = 0;; j += 3) {
    load(s2, min(j + 2, last));
    __builtin_amdgcn_sched_barrier(0);
    mul(s0);
    __builtin_amdgcn_sched_barrier(0);
    if (j + 1 >= steps) break;
    load(s0, min(j + 3, last));
    __builtin_amdgcn_sched_barrier(0);
    mul(s1);
    __builtin_amdgcn_sched_barrier(0);
    if (j + 2 >= steps) break;
    load(s1, min(j + 4, last));
    __builtin_amdgcn_sched_barrier(0);
    mul(s2);
    __builtin_amdgcn_sched_barrier(0);
    if (j + 3 >= steps) break;
  }
  // D[i][jj]: jj = lane % 32 (weight row), i = 8 (v / 4) + 4 (lane / 32) + v % 4 (token)
#pragma unroll
  for (int m = 0; m < MATS; ++m)
#pragma unroll
    for (int v = 0; v < 16; ++v) part[m][wave][8 * (v >> 2) + 4 * h + (v & 3)][r] = acc[m][v];
  __syncthreads();
  for (int idx = threadIdx.x; idx < 32 * 32; idx += NW * 64) {
    const int rr = idx & 31, t = idx >> 5;  // consecutive threads: consecutive rows of one token
    const int row = row0 + rr;
    if (row >= a.rows || t >= a.tokens) continue;
    float y[MATS];
#pragma unroll
    for (int m = 0; m < MATS; ++m) {
      float sum = part[m][0][t][rr];
#pragma unroll
      for (int w = 1; w < NW; ++w) sum += part[m][w][t][rr];
      y[m] = sum;
    }
    const size_t o = (size_t)t * a.out_stride + row;
    if (DUAL) {
      ((uint16_t *)a.out)[o] = kx_bf16_rne(kx_swiglu(kx_bfround(y[0]), kx_bfround(y[MATS - 1])));
    } else if (a.mode == KX_GG_BF16) {
      ((uint16_t *)a.out)[o] = kx_bf16_rne(y[0]);
    } else if (a.mode == KX_GG_F32) {
      ((float *)a.out)[o] = y[0];
    } else if (a.mode == KX_GG_F32_OF_BF16) {
      ((float *)a.out)[o] = kx_bfround(y[0]);
    } else {  // x = bf(x + bf(y))  (add_k, :248-251)
      uint16_t *xo = (uint16_t *)a.out + o;
      *xo = kx_bf16_rne(kx_bf16_f32(*xo) + kx_bfround(y[0]));
    }
  }
}

}  // namespace

// One tile of up to 32 tokens against a bf16 matrix (two for SwiGLU).  Returns KX_OK with *done = false, having
// launched nothing, when the shape is not the kernel's (cols not a multiple of 512, more than 32 tokens).
int kx_skinny_gemm_launch(bool dual, const uint16_t *w0, const uint16_t *w1, const uint16_t *x, int x_stride, void *out,
                          int out_stride, int out_mode, int tokens, int rows, int cols, bool *done, hipStream_t st) {
  *done = false;
  if (tokens < 1 || tokens > 32 || rows < 1 || cols < 512 || cols % 512 || x_stride % 8 || (dual && !w1)) return KX_OK;
  KX_REQUIRE(out_mode >= KX_GG_BF16 && out_mode <= KX_GG_RESID && !(dual && out_mode != KX_GG_BF16), "kx_skinny_gemm: out_mode=%d", out_mode);
  SkinnyArgs a;
  a.w0 = w0; a.w1 = w1; a.x = x; a.out = out; a.rows = rows; a.cols = cols; a.tokens = tokens; a.x_stride = x_stride;
  a.out_stride = out_stride; a.mode = out_mode;
  const dim3 g((unsigned)kx_cdiv(rows, 32));
  // eight waves: with 12 or 16 (where they divide the columns) the same matrices take 1.2-1.4 times as long
  if (dual) hipLaunchKernelGGL((skinny_gemm_k<true, 8>), g, dim3(512), 0, st, a);
  else hipLaunchKernelGGL((skinny_gemm_k<false, 8>), g, dim3(512), 0, st, a);
  KX_LAUNCH_CHECK();
  *done = true;
  return KX_OK;
}
