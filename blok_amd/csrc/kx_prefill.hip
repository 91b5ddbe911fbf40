// kx_prefill.hip -- W4A16 grouped GEMM for prefill chunks through one MoE layer.
//
// The reference has no batched prefill: it runs one decode step per prompt token
// (src/kimi_exec.cu:886) and, inside it, the per-expert loops at :845-870.  For a
// chunk of T tokens this file computes the same per-token quantities -- gate/up
// projections with SwiGLU (:853-862), down projection (:863-869), the routed
// combine (:868,:871), the shared expert (:872-875) and the residual add (:877) --
// with the tokens of each expert gathered into one GEMM.
//
// The only place MFMA is used.  Per workgroup (8 waves): one expert, 256 weight rows, the
// expert's tokens in tiles of 128.  Wave w owns weight rows 32 w .. +31 for all 128 tokens
// (fp32 accumulators of v_mfma_f32_32x32x16_bf16).  Per K step of 64 columns:
//  * INT4 weights reach the lanes through LDS as packed words: for every two K steps the
//    64-byte runs of the 256 rows (both matrices) are copied by global -> LDS loads, which
//    take no registers and use every byte they fetch, into a ring of two stages; lane
//    (r, h) = (lane % 32, lane / 32) reads the 16 bytes of row r that hold columns 32 h .. +31
//    of the step -- one quantization group, four packed words -- and dequantizes word j to
//    the reference's values, w = bf((n-8)*scale) (:311-312), which is exactly the B operand
//    of the step's j-th MFMA when that MFMA contracts over columns {8 j .. +7} and
//    {32 + 8 j .. +7} (the contraction order within a step is free, the activation operand
//    uses the same columns).  The 16-byte pieces of a row are stored xor-swizzled by the row
//    so that the lanes' reads are free of bank conflicts.  Group scales are copied to LDS
//    the same way, sixteen K steps at a time: 64 bytes per row and matrix, a whole sector of the row (blocks of
//    eight steps fetched half of every sector twice);
//  * bf16 weights (shared expert, router gate) are loaded by the lanes themselves, 64
//    contiguous bytes per lane and step, one step ahead;
//  * the gathered activation rows go through a double-buffered LDS tile, one barrier per step; with INT4
//    weights they are copied global -> LDS as well (128-byte rows, pieces xor-swizzled by the row), with bf16
//    weights they pass through registers into rows padded to 144 bytes.
//
// Dequant without integer conversion: (w & 0x000F000F) | 0x64006400 is the f16 pair
// (1024+n0, 1024+n4), (w & 0x00F000F0) | 0x64006400 is (1024+16 n1, 1024+16 n5), w >> 8 gives
// n2,n6,n3,n7 the same way; fma(f16, s, -1032 s) = (n-8) s and fma(f16, s/16, -72 s) = (n-8) s
// are exact in fp32 (4-bit times 8-bit significands), and one v_cvt_pk_bf16_f32 rounds two of
// them to nearest-even.
//
// MFMA's internal summation order is not documented, so this path is held to the
// max-rel 1e-2 bar and is never used for the token-identity runs.
#include <atomic>
#include "kx_common.h"
#include "kx_lds_copy.h"
#include "kx_dense.h"
#include "kx_math.h"

#include <type_traits>

namespace {

typedef __bf16 kx_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 kx_bf16x2 __attribute__((ext_vector_type(2)));
typedef float kx_f32x2 __attribute__((ext_vector_type(2)));
typedef float kx_f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 kx_h2 __attribute__((ext_vector_type(2)));

constexpr int BN = 256, BK = 64;  // a token tile has up to 4 blocks of 32 tokens (PfArgs::nb_max)
constexpr int LDS_STRIDE = BK + 8;  // bf16 elements per LDS row: 144 B keeps 16-byte reads of a column of rows spread over banks
constexpr int W_STAGE = BN * 64;               // bytes of one matrix's packed words for two K steps
constexpr int SC_BLOCK = 16;                   // K steps per staged block of group scales
constexpr int SC_STRIDE = SC_BLOCK * 4;        // bytes per (row, matrix) of a block: 32 bf16, one 64-byte sector of the row

struct PfArgs {
  const void *w0, *w1;          // INT4: packed i32 [E][N][K/8]; BF16: bf16 [E][N][K]
  const uint16_t *s0, *s1;      // INT4: bf16 scales [E][N][K/32]
  const uint16_t *x;            // bf16 activation rows of K
  void *out;                    // bf16 [pairs][N], or f32 (see out_mode)
  const int4 *work;             // {expert, first, last, _} per expert with work; nullptr: one group of n_pairs rows
  const int *pairs;             // pair ids sorted by expert; nullptr: identity
  int n_pairs, N, K, x_div;     // activation row = pair / x_div
  size_t expert_w, expert_s;    // elements between experts (words or bf16; scales)
  int out_mode;                 // single matrix only: KX_GG_BF16, KX_GG_F32, KX_GG_F32_OF_BF16 or KX_GG_RESID
  int nb_max;                   // 32-token blocks per token tile (1..4): sizes the activation tiles in LDS
  int cnt_lo;                   // groups with fewer pairs are left to another launch
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

// The INT4 kernels keep copies and loads in flight across barriers and LDS accesses, and say themselves when
// one has to have landed.  The compiler would not let them: it completes every global -> LDS copy in flight
// (s_waitcnt vmcnt(0)) in front of an LDS access it cannot tell from the copy's target and in front of every
// fenced barrier, and loads complete in order, so a wait for a plain load it issued waits for the copies too.
// Hence: weights and activations both reach LDS by copies issued from inline asm (unknown to the compiler), the
// barrier has no fence, and the waits are explicit and counted.
__device__ __forceinline__ void pf_copy16_to_lds(const void *src, uint32_t lds_base) {
  kx_copy16_to_lds(src, __builtin_amdgcn_readfirstlane(lds_base));
}
template <int N>
__device__ __forceinline__ void pf_wait_copies() { kx_wait_copies<N>(); }
__device__ __forceinline__ void pf_barrier() { kx_lds_barrier(); }

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

// WAVES waves per workgroup, 32 weight rows each (INT4: 8, the ring and the scale staging are laid out for 256 rows)
template <bool DUAL, bool I4, int WAVES>
__global__ void __launch_bounds__(WAVES * 64, (I4 || WAVES < 8) ? 1 : 2) grouped_gemm_k(PfArgs a) {
  static_assert(!I4 || WAVES == 8, "the INT4 path is laid out for 8 waves");
  constexpr int MATS = DUAL ? 2 : 1;
  extern __shared__ __attribute__((aligned(16))) uint8_t pf_lds[];
  const int BM = a.nb_max * 32, XT = BM * (I4 ? BK : LDS_STRIDE);  // tokens and elements of one activation tile
  uint16_t *xs_lds = (uint16_t *)pf_lds;                 // two activation tiles
  uint8_t *w_ring = pf_lds + 2 * XT * 2;                 // INT4: [2 stages][MATS][256 rows][4 pieces of 16 B]
  uint8_t *sc_lds = w_ring + 2 * MATS * W_STAGE;         // INT4: [2 blocks][MATS][256 rows][SC_STRIDE]
  const uint32_t ring0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)w_ring;  // LDS address of the ring
  const uint32_t sc0 = ring0 + 2 * MATS * W_STAGE;                                                  // of the scale blocks
  const uint32_t xs0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)pf_lds;    // and of the activation tiles
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 31, lh = lane >> 5;
  const int n0 = blockIdx.x * (WAVES * 32);
  int4 wk = a.work ? a.work[blockIdx.y] : make_int4(0, 0, a.n_pairs, 0);
  const int e = __builtin_amdgcn_readfirstlane(wk.x);
  if (e < 0) return;
  const int p_begin = __builtin_amdgcn_readfirstlane(wk.y), p_end = __builtin_amdgcn_readfirstlane(wk.z);
  if (p_end - p_begin < a.cnt_lo) return;
  uint32_t magic;
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));
  const int nk = a.K / BK;
  const int trow = wave * 32 + lr;                       // this lane's weight row within the tile
  const int wrow = min(n0 + trow, a.N - 1);
  // bf16 weights: this lane's row and its 32-column half of every K step
  const uint16_t *wb_ptr[MATS];
#pragma unroll
  for (int m = 0; m < MATS; ++m)
    wb_ptr[m] = (const uint16_t *)(m ? a.w1 : a.w0) + (size_t)e * a.expert_w + (size_t)wrow * a.K + lh * 32;
  // INT4: global -> LDS copies of this wave for one stage: MATS*2 instructions of 64 pieces
  const uint32_t *dma_src[MATS * 2];
  int dma_dst[MATS * 2];
#pragma unroll
  for (int u = 0; u < MATS * 2; ++u) {
    const int g = (wave * MATS * 2 + u) * 64 + lane;     // piece index over [MATS][256 rows][4]
    const int m = g >> 10, sl = g & 1023, row = sl >> 2, ps = sl & 3;
    const int p = ps ^ ((row >> 2) & 3);                 // the piece of the row that lives in slot ps
    dma_src[u] = (const uint32_t *)(m ? a.w1 : a.w0) + (size_t)e * a.expert_w + (size_t)min(n0 + row, a.N - 1) * (a.K >> 3) + p * 4;
    dma_dst[u] = (wave * MATS * 2 + u) * 1024;           // byte offset within a stage, the same for the whole wave
  }
  auto dma_stage = [&](int ss) {  // packed words of K steps 2 ss, 2 ss + 1 into stage ss % 2
    if (I4) {
#pragma unroll
      for (int u = 0; u < MATS * 2; ++u)
        pf_copy16_to_lds(dma_src[u] + ss * 16, ring0 + (ss & 1) * MATS * W_STAGE + dma_dst[u]);
    }
  };
  // group scales: blocks of SC_BLOCK K steps, 64 bytes per row and matrix -- whole sectors -- copied global -> LDS.
  // Instruction c = wave * 2 MATS + i covers pieces 64 c .. +63 of [MATS][256 rows][4 slots]; slot s of row r holds
  // piece s ^ ((r / 2) % 4): a wave reads one 2-byte scale per row at the same offset of 32 consecutive rows, and with
  // the pieces in place (64-byte rows) those fall into two banks; xor-ed by the row they fall into eight.  A last block of
  // half the steps (K / 64 an odd multiple of 8) repeats its two pieces, the copies land in slots that are never read.
  const uint16_t *sc_src[MATS * 2];
#pragma unroll
  for (int i = 0; i < MATS * 2; ++i) {
    const int c = wave * MATS * 2 + i, m = c >> 4, row = (c & 15) * 16 + (lane >> 2);
    sc_src[i] = (m ? a.s1 : a.s0) + (I4 ? (size_t)e * a.expert_s + (size_t)min(n0 + row, a.N - 1) * (a.K >> 5) : 0);
  }
  auto copy_scales = [&](int blk) {
    if (I4) {
      const int left = (nk - blk * SC_BLOCK) >> 2;  // 16-byte pieces of the row from this block on: 2 or at least 4
      const int piece = min((lane & 3) ^ ((lane >> 3) & 3), left - 1);  // row = 16 (c % 16) + lane / 4
#pragma unroll
      for (int i = 0; i < MATS * 2; ++i)
        pf_copy16_to_lds(sc_src[i] + blk * (SC_BLOCK * 2) + piece * 8,
                         sc0 + (blk & 1) * (BN * MATS * SC_STRIDE) + (wave * MATS * 2 + i) * 1024);
    }
  };
  // activation staging: thread -> rows tid/4 + q * (16 WAVES), 16 columns from (tid%4)*16
  constexpr int XROWS = WAVES * 16;  // rows staged per pass of the workgroup
  const int xr = tid >> 2, xc = (tid & 3) * 16;

  for (int m0 = p_begin + blockIdx.z * BM; m0 < p_end; m0 += gridDim.z * BM) {
    const int nb = min(a.nb_max, (p_end - m0 + 31) >> 5);  // 32-token blocks that hold tokens
    constexpr int XQMAX = (128 + XROWS - 1) / XROWS;
    const uint16_t *xrow[XQMAX];
    bool x_valid[XQMAX];
#pragma unroll
    for (int q = 0; q < XQMAX; ++q) {
      const int pi = m0 + q * XROWS + xr;
      x_valid[q] = pi < p_end && q * XROWS + xr < a.nb_max * 32;
      const int pair = x_valid[q] ? (a.pairs ? a.pairs[pi] : pi) : 0;
      xrow[q] = a.x + (size_t)(pair / a.x_div) * a.K + xc;
    }

    // INT4 path: the activation tile goes global -> LDS like the weights.  A row of a K step is 128 B = 8 pieces;
    // copy instruction ii covers rows 8 ii .. 8 ii + 7, slot (row, p') holding piece p' ^ ((row >> 1) & 7), so that
    // the row-per-lane operand reads are free of bank conflicts without padding.  Rows past the expert's tokens
    // read pair 0: they only feed accumulator rows that are never stored.
    constexpr int XCMAX = 2;  // copy instructions per wave and K step at 128 tokens
    const uint16_t *xc_src[XCMAX];
    int xc_dst[XCMAX];
    if (I4) {
#pragma unroll
      for (int q = 0; q < XCMAX; ++q) {
        const int ii = min(wave + 8 * q, a.nb_max * 4 - 1);
        const int slot = ii * 64 + lane, row = slot >> 3, piece = (slot & 7) ^ ((row >> 1) & 7);
        const int pi = m0 + row;
        const int pair = pi < p_end ? (a.pairs ? a.pairs[pi] : pi) : 0;
        xc_src[q] = a.x + (size_t)(pair / a.x_div) * a.K + piece * 8;
        xc_dst[q] = ii * 1024;
      }
    }

    // the tile with NB token blocks, NB a compile-time constant so that the K loop has no branches
    auto run = [&](auto nb_c) {
      constexpr int NB = decltype(nb_c)::value;
      kx_f32x16 acc[MATS][NB];
#pragma unroll
      for (int m = 0; m < MATS; ++m)
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[m][t][i] = 0.0f;
      struct WRaw {
        uint4 q[MATS];              // INT4: the group's four packed words
        float sc[MATS];
        uint4 b[MATS][I4 ? 1 : 4];  // BF16: 32 columns
      };
      constexpr int XQ = (NB * 32 + XROWS - 1) / XROWS;  // staging passes that hold rows of this tile
      uint4 xv[XQ][2];
      auto load_x = [&](int ks) {  // bf16 weights: activations through registers
#pragma unroll
        for (int q = 0; q < XQ; ++q) {
          xv[q][0] = xv[q][1] = make_uint4(0, 0, 0, 0);
          if (x_valid[q] && q * XROWS + xr < NB * 32) {
            xv[q][0] = *(const uint4 *)(xrow[q] + ks * BK);
            xv[q][1] = *(const uint4 *)(xrow[q] + ks * BK + 8);
          }
        }
      };
      auto store_x = [&](uint16_t *st) {
#pragma unroll
        for (int q = 0; q < XQ; ++q)
          if (q * XROWS + xr < NB * 32) {
            *(uint4 *)(st + (q * XROWS + xr) * LDS_STRIDE + xc) = xv[q][0];
            *(uint4 *)(st + (q * XROWS + xr) * LDS_STRIDE + xc + 8) = xv[q][1];
          }
      };
      constexpr int XC = (NB * 4 + 7) / 8;  // INT4: activation copies per wave and K step (every wave issues XC)
      auto copy_x = [&](int ks) {            // activations of K step ks into tile ks % 2
#pragma unroll
        for (int q = 0; q < XC; ++q) pf_copy16_to_lds(xc_src[q] + ks * BK, xs0 + (ks & 1) * XT * 2 + xc_dst[q]);
      };
      // this lane's weights of K step ks: INT4 from the LDS ring and the staged scales, bf16 from memory
      auto fetch_w = [&](WRaw &r, int ks) {
#pragma unroll
        for (int m = 0; m < MATS; ++m) {
          if (I4) {
            const int q = (ks & 1) * 2 + lh;
            const uint8_t *st = w_ring + ((ks >> 1) & 1) * MATS * W_STAGE + m * W_STAGE;
            r.q[m] = *(const uint4 *)(st + (trow * 4 + (q ^ ((trow >> 2) & 3))) * 16);
            const uint8_t *sb = sc_lds + ((ks / SC_BLOCK) & 1) * (BN * MATS * SC_STRIDE) + (m * BN + trow) * SC_STRIDE;
            const int el = (ks % SC_BLOCK) * 2 + lh;  // the lane's group among the block's 32
            r.sc[m] = kx_bf16_f32(*(const uint16_t *)(sb + (((el >> 3) ^ ((trow >> 1) & 3)) * 8 + (el & 7)) * 2));
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) r.b[m][j] = *(const uint4 *)(wb_ptr[m] + ks * BK + j * 8);
          }
        }
      };
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
        if (I4) {  // 128-byte rows, pieces xor-swizzled by the row
          const int off = lr * 128 + (((lh * 4 + j) ^ (lr >> 1)) & 7) * 16;
#pragma unroll
          for (int t = 0; t < NB; ++t) av[t] = *(const kx_bf16x8 *)((const uint8_t *)xs + t * 32 * 128 + off);
        } else {
          const int kcol = lh * 32 + j * 8;
#pragma unroll
          for (int t = 0; t < NB; ++t) av[t] = *(const kx_bf16x8 *)(xs + (t * 32 + lr) * LDS_STRIDE + kcol);
        }
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
      // one K step.  MFMA j contracts over columns 8 j .. +7 (lanes 0-31) and 32 + 8 j .. +7 (lanes 32-63); the
      // operands of group j+1 (LDS reads, dequant) are produced while the matrix cores run group j.
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

      // prologue: stage 0 of the ring, the first scale block, the first activation tile
      auto barrier = [&]() {
        if (I4) pf_barrier();
        else __syncthreads();
      };
      WRaw w0, w1;
      if (I4) {
        copy_scales(0);
        copy_x(0);
        dma_stage(0);
      } else {
        load_x(0);
        fetch_w(w0, 0);
      }
      if (!I4) store_x(xs_lds);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      barrier();
      for (int ks = 0; ks < nk; ks += 2) {
        // even step: the other ring stage and the other activation tile were last read behind a barrier.  Order of
        // issue: activations of the next step, the ring copies, then (every SC_BLOCK steps) the next scale block; the
        // activations have to land by the end of this step, the copies behind them stay in flight until the end of
        // the odd step (a wave's copies complete in the order of issue)
        const bool scales_now = I4 && ks % SC_BLOCK == 0 && ks + SC_BLOCK < nk;
        if (I4) {
          if (ks + 1 < nk) copy_x(ks + 1);
          if (ks + 2 < nk) dma_stage((ks >> 1) + 1);
          if (scales_now) copy_scales(ks / SC_BLOCK + 1);
          fetch_w(w0, ks);
        } else {
          if (ks + 1 < nk) load_x(ks + 1);
          if (ks + 1 < nk) fetch_w(w1, ks + 1);
        }
        step(w0, ks);
        if (I4) {
          if (scales_now) pf_wait_copies<MATS * 4>();
          else if (ks + 2 < nk) pf_wait_copies<MATS * 2>();
          else pf_wait_copies<0>();
        } else if (ks + 1 < nk) {
          store_x(xs_lds + XT);
        }
        barrier();
        if (ks + 1 < nk) {
          if (I4) {
            if (ks + 2 < nk) copy_x(ks + 2);
            fetch_w(w1, ks + 1);
          } else {
            if (ks + 2 < nk) load_x(ks + 2);
            if (ks + 2 < nk) fetch_w(w0, ks + 2);
          }
          step(w1, ks + 1);
          if (!I4 && ks + 2 < nk) store_x(xs_lds);
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's copies (ring stage, activations) have landed
          barrier();
        }
      }
      // epilogue: D[i][j], j = lane % 32 (weight row), i = 8*(v/4) + 4*(lane/32) + v%4 (token of the 32-token block)
      const int n = n0 + trow;
      if (n < a.N) {
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int po = m0 + t * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
            if (po < p_end) {
              const int pr = a.pairs ? a.pairs[po] : po;
              float r = acc[0][t][v];
              if (DUAL) r = kx_swiglu(kx_bfround(r), kx_bfround(acc[MATS - 1][t][v]));
              if (DUAL || a.out_mode == KX_GG_BF16) {
                ((uint16_t *)a.out)[(size_t)pr * a.N + n] = kx_bf16_rne(r);
              } else if (a.out_mode == KX_GG_F32) {
                ((float *)a.out)[(size_t)pr * a.N + n] = r;
              } else if (a.out_mode == KX_GG_F32_OF_BF16) {
                ((float *)a.out)[(size_t)pr * a.N + n] = kx_bfround(r);
              } else {  // x = bf(x + bf(y))  (add_k, :248-251)
                uint16_t *xo = (uint16_t *)a.out + (size_t)pr * a.N + n;
                *xo = kx_bf16_rne(kx_bf16_f32(*xo) + kx_bfround(r));
              }
            }
          }
      }
      __syncthreads();  // the next token tile starts by overwriting the LDS tiles
    };
    if (nb == 1) run(std::integral_constant<int, 1>{});
    else if (nb == 2 || !I4) run(std::integral_constant<int, 2>{});  // bf16 weights are launched with nb_max 2
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
                           const uint16_t *x, void *out, int out_mode, const int4 *work, const int *pairs, int n_pairs,
                           int n_slots, int N, int K, int x_div, size_t expert_w, size_t expert_s, int n_pairs_max,
                           hipStream_t st, int cnt_lo) {
  KX_REQUIRE(K > 0 && K % 128 == 0 && (!i4 || K % 512 == 0), "kx_grouped_gemm: K=%d must be a positive multiple of %d", K, i4 ? 512 : 128);
  KX_REQUIRE(N > 0, "kx_grouped_gemm: N=%d must be positive", N);
  KX_REQUIRE(out_mode >= KX_GG_BF16 && out_mode <= KX_GG_RESID && !(dual && out_mode != KX_GG_BF16), "kx_grouped_gemm: out_mode=%d", out_mode);
  PfArgs a;
  a.w0 = w0; a.w1 = w1; a.s0 = s0; a.s1 = s1; a.x = x; a.out = out; a.work = work; a.pairs = pairs;
  a.n_pairs = n_pairs; a.N = N; a.K = K; a.x_div = x_div; a.expert_w = expert_w; a.expert_s = expert_s;
  a.out_mode = out_mode;
  a.cnt_lo = cnt_lo;
  // token tile: 128 tokens for the INT4 kernels, whose dequant work per weight tile is amortised over the tokens;
  // 64 for the bf16 ones (more workgroups for the one-group GEMMs of the shared expert and the router)
  a.nb_max = i4 ? 4 : 2;
  const int BM = a.nb_max * 32;
  const int max_rows = work ? n_pairs_max : n_pairs;
  int mz = kx_cdiv(max_rows, BM);
  mz = mz < 1 ? 1 : mz > 64 ? 64 : mz;
  // waves per workgroup (32 weight rows each): 8 for INT4; for bf16 as few as it takes to get a couple of hundred
  // workgroups (a decode batch is one token tile, so the N rows are the only source of parallelism there)
  const long tiles = (long)mz * (work ? n_slots : 1);
  const int waves = i4 ? 8 : (N / 256 * tiles >= 192 ? 8 : N / 64 * tiles >= 192 ? 2 : 1);
  dim3 g(kx_cdiv(N, waves * 32), work ? n_slots : 1, mz), b(waves * 64);
  const int mats = dual ? 2 : 1;
  const size_t lds = (size_t)2 * BM * (i4 ? BK : LDS_STRIDE) * 2 + (i4 ? (size_t)2 * mats * W_STAGE + (size_t)2 * BN * mats * SC_STRIDE : 0);
  static std::atomic<bool> attr_set{false};  // setting it twice from two threads is harmless
  if (!attr_set) {  // more than 64 KB of dynamic LDS has to be allowed per kernel
    KX_HIP(hipFuncSetAttribute((const void *)grouped_gemm_k<true, true, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)grouped_gemm_k<false, true, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    attr_set = true;
  }
#define KX_GG(D, W) hipLaunchKernelGGL((grouped_gemm_k<D, false, W>), g, b, lds, st, a)
  if (dual && i4) hipLaunchKernelGGL((grouped_gemm_k<true, true, 8>), g, b, lds, st, a);
  else if (i4) hipLaunchKernelGGL((grouped_gemm_k<false, true, 8>), g, b, lds, st, a);
  else if (dual) { if (waves == 8) KX_GG(true, 8); else if (waves == 2) KX_GG(true, 2); else KX_GG(true, 1); }
  else { if (waves == 8) KX_GG(false, 8); else if (waves == 2) KX_GG(false, 2); else KX_GG(false, 1); }
#undef KX_GG
  KX_LAUNCH_CHECK();
  return KX_OK;
}

int kx_moe_combine_launch(const uint16_t *eout, const float *rw, const uint16_t *sy, uint16_t *x, int tokens, int hidden,
                          int topk, uint32_t flags, hipStream_t st) {
  hipLaunchKernelGGL(moe_combine_k, dim3(kx_cdiv(hidden, 256), tokens), dim3(256), 0, st, eout, rw, sy, x, hidden, topk, flags);
  KX_LAUNCH_CHECK();
  return KX_OK;
}
