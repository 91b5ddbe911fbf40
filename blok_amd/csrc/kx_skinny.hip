// kx_skinny.hip -- dense projections for decode batches of 5 to 32 sequences: y[t, r] = sum_k x[t, k] w[r, k] with
// bf16 weights [rows, cols] streamed once and the tokens as the other side of a matrix-core product.
//
// Reference: matvec_bf16_k / matvec_bf16_f32_k (src/kimi_exec.cu:272-298) called once per token; the epilogues are
// add_k (:248-251), silu_mul_k (:253-256) and the bf16 rounding of the logits (:718-734).
//
// A GEMV kernel streams the weights once per block of four tokens and is bound by its fma count from about 16 tokens
// on (every weight meets every token on the VALU), and
// the grouped prefill GEMM of kx_prefill.hip, built for 128-token tiles of many experts, leaves most of the chip idle
// on one 32-token tile.  Here a workgroup of 8 waves owns 32 weight rows and all (up to 32) tokens, the eight waves
// split the columns, and their partial 32 x 32 tiles (v_mfma_f32_32x32x16_bf16) are summed through LDS in wave
// order before the epilogue.
//
// Both operands are staged through LDS.  The operand layout of the matrix cores is one row per lane: loading the
// operands straight from memory makes every load instruction touch 32 rows with 32 bytes each, and that streams at
// 2.3-3 TB/s whatever the number of waves (measured; the lm_head then takes 1.0 ms).  So the columns are walked in
// blocks of 256: a copy instruction (global_load_lds_dwordx4, no registers) moves 512 contiguous bytes of two rows,
// lane (l / 32, l % 32) = (row of the pair, 16-byte slot); the lane fetches piece slot ^ (row % 16) of its row, so
// that the operand reads -- lane (r, h) wants piece p of row r and finds it in slot p ^ (r % 16) -- fall into different
// banks.  Blocks go through a ring of 4 stages (3 for two matrices), three (two) blocks in flight behind the one being
// multiplied; each wave issues its share of a block's copies, waits for its own by count (they complete in order),
// and one barrier per block makes every wave's copies visible and the stage that is overwritten next free.  Wave w
// multiplies pieces 4w .. 4w+3 of the block (two products per matrix).  The lm_head takes 0.43 ms this way (5.5 TB/s).
// The copies are issued from inline asm and the barrier carries no fence: a copy the compiler knows of makes it
// complete everything in flight before every LDS access it cannot tell from the copy's target.
//
// Sums are fp32 over exact bf16 products in another order than the GEMV's: this path is held to the 1e-2 bar, like the
// other matrix-core paths, and serves batches the token-identity checks do not run on.
#include <atomic>
#include "kx_common.h"
#include "kx_lds_copy.h"
#include "kx_dense.h"
#include "kx_math.h"

namespace {

typedef __bf16 kx_bf16x8 __attribute__((ext_vector_type(8)));
typedef float kx_f32x16 __attribute__((ext_vector_type(16)));

struct SkinnyArgs {
  const uint16_t *w0, *w1;  // bf16 [rows, cols]; w1 for the two-matrix SwiGLU form
  const uint16_t *x;        // bf16 [tokens, x_stride]
  void *out;                // [tokens, out_stride]: bf16, or f32 (see mode)
  int rows, cols, tokens, x_stride, out_stride, mode;
};

__device__ __forceinline__ void sk_copy16_to_lds(const void *src, uint32_t lds_base) {
  kx_copy16_to_lds(src, __builtin_amdgcn_readfirstlane(lds_base));
}
template <int N>
__device__ __forceinline__ void sk_wait_copies() { kx_wait_copies<N>(); }
__device__ __forceinline__ void sk_barrier() { kx_lds_barrier(); }

template <bool DUAL>
__global__ void __launch_bounds__(512) skinny_staged_k(SkinnyArgs a) {
  constexpr int MATS = DUAL ? 2 : 1;
  constexpr int TILES = MATS + 1;            // weight tiles and the activation tile of a stage, 16 KB each
  constexpr int NS = DUAL ? 3 : 4;           // stages
  constexpr int CPW = TILES * 2;             // copy instructions per wave and block (16 per tile over 8 waves)
  constexpr uint32_t TILE = 32 * 512, STAGE = TILES * TILE;
  extern __shared__ __attribute__((aligned(16))) uint8_t sk_lds[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)sk_lds;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 31, h = lane >> 5;
  const int row0 = blockIdx.x * 32;
  const int nb = a.cols >> 8;  // blocks of 256 columns
  // this wave's copies of a block: instruction u moves rows 2 i, 2 i + 1 of tile t, (t, i) = ((8 u + wave) / 16, .. % 16)
  const uint16_t *csrc[CPW];
  uint32_t cdst[CPW];
#pragma unroll
  for (int u = 0; u < CPW; ++u) {
    const int idx = u * 8 + wave, t = idx >> 4, i = idx & 15;
    const int row = 2 * i + h, piece = r ^ (row & 15);
    const uint16_t *base = t == MATS ? a.x + (size_t)min(row, a.tokens - 1) * a.x_stride
                                     : (t == 0 ? a.w0 : a.w1) + (size_t)min(row0 + row, a.rows - 1) * a.cols;
    csrc[u] = base + piece * 8;
    cdst[u] = t * TILE + i * 1024;
  }
  auto copy_block = [&](int b) {
    const uint32_t st = lds0 + (uint32_t)(b % NS) * STAGE;
#pragma unroll
    for (int u = 0; u < CPW; ++u) sk_copy16_to_lds(csrc[u] + b * 256, st + cdst[u]);
  };
  kx_f32x16 acc[MATS];
#pragma unroll
  for (int m = 0; m < MATS; ++m)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[m][v] = 0.0f;
  // operand reads of this lane: piece 4 wave + 2 q + h of row r sits in slot piece ^ (r % 16)
  uint32_t roff[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) roff[q] = (uint32_t)r * 512 + (uint32_t)((4 * wave + 2 * q + h) ^ (r & 15)) * 16;

#pragma unroll
  for (int b = 0; b < NS - 1; ++b)
    if (b < nb) copy_block(b);
  for (int b = 0; b < nb; ++b) {
    // this wave's copies of block b have landed when at most those of the blocks behind it are in flight
    const int behind = min(nb - 1 - b, NS - 2);
    if (behind >= 2) sk_wait_copies<2 * CPW>();
    else if (behind == 1) sk_wait_copies<CPW>();
    else sk_wait_copies<0>();
    sk_barrier();  // every wave's copies of block b are in LDS; every wave is done with block b - 1
    if (b + NS - 1 < nb) copy_block(b + NS - 1);  // into the stage block b - 1 was read from
    const uint8_t *st = sk_lds + (uint32_t)(b % NS) * STAGE;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const kx_bf16x8 xv = *(const kx_bf16x8 *)(st + MATS * TILE + roff[q]);
#pragma unroll
      for (int m = 0; m < MATS; ++m) {
        const kx_bf16x8 wv = *(const kx_bf16x8 *)(st + m * TILE + roff[q]);
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xv, wv, acc[m], 0, 0, 0);
      }
    }
  }
  sk_barrier();  // the ring is free: it takes the partial tiles
  float(*part)[8][32][32] = (float(*)[8][32][32])sk_lds;
#pragma unroll
  for (int m = 0; m < MATS; ++m)
#pragma unroll
    for (int v = 0; v < 16; ++v) part[m][wave][8 * (v >> 2) + 4 * h + (v & 3)][r] = acc[m][v];
  __syncthreads();
  for (int idx = threadIdx.x; idx < 32 * 32; idx += 512) {
    const int rr = idx & 31, t = idx >> 5;
    const int row = row0 + rr;
    if (row >= a.rows || t >= a.tokens) continue;
    float y[MATS];
#pragma unroll
    for (int m = 0; m < MATS; ++m) {
      float sum = part[m][0][t][rr];
#pragma unroll
      for (int w = 1; w < 8; ++w) sum += part[m][w][t][rr];
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
  if (tokens < 1 || tokens > 32 || rows < 1 || cols < 512 || cols % 512 || x_stride % 8 || x_stride < cols || (dual && !w1)) return KX_OK;
  KX_REQUIRE(out_mode >= KX_GG_BF16 && out_mode <= KX_GG_RESID && !(dual && out_mode != KX_GG_BF16), "kx_skinny_gemm: out_mode=%d", out_mode);
  SkinnyArgs a;
  a.w0 = w0; a.w1 = w1; a.x = x; a.out = out; a.rows = rows; a.cols = cols; a.tokens = tokens; a.x_stride = x_stride;
  a.out_stride = out_stride; a.mode = out_mode;
  const dim3 g((unsigned)kx_cdiv(rows, 32));
  const size_t lds = (size_t)(dual ? 3 * 3 : 4 * 2) * 32 * 512;  // the ring: stages x tiles x 16 KB
  static std::atomic<bool> attr{false};  // setting it twice from two threads is harmless
  if (!attr) {
    KX_HIP(hipFuncSetAttribute((const void *)skinny_staged_k<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 4 * 2 * 32 * 512));
    KX_HIP(hipFuncSetAttribute((const void *)skinny_staged_k<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 3 * 3 * 32 * 512));
    attr = true;
  }
  if (dual) hipLaunchKernelGGL(skinny_staged_k<true>, g, dim3(512), lds, st, a);
  else hipLaunchKernelGGL(skinny_staged_k<false>, g, dim3(512), lds, st, a);
  KX_LAUNCH_CHECK();
  *done = true;
  return KX_OK;
}
