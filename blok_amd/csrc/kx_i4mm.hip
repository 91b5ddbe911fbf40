// kx_i4mm.hip -- W4A16 products of the routed experts for a few tokens per expert (3 to 32: a decode batch's experts
// that several sequences share), on the matrix cores, with the weights dequantized in registers.
//
// The reference runs one GEMV per (token, expert) (src/kimi_exec.cu:845-870); the GEMV kernels of kx_i4.hip stream
// an expert's weights once per token of it, the grouped GEMM of kx_prefill.hip once per 128-token tile but at 1.3 us
// per K step whatever the tokens.  Here a wave owns 32 weight rows (of both matrices for gate/up) and goes over all
// columns, 256 at a time (128 bytes of a row):
//  * the 32 x 128 bytes are loaded as whole lines, eight lanes per row (four instructions of 1 KB), two runs ahead,
//    and turned into the row-per-lane layout of the MFMA operand through a 4 KB tile of LDS that belongs to the
//    wave alone -- no workgroup barrier, the LDS pipeline keeps a wave's operations in order; 16-byte pieces
//    xor-ed by the row, so neither side has bank conflicts.  (Loading row-per-lane straight from memory, 16 bytes
//    per lane, asked for every 128-byte line eight times and streamed at 0.8 TB/s.)
//  * lane (r, h) = (lane % 32, lane / 32) then holds columns 128 h .. +127 of row r: four quantization groups of four
//    packed words, and each word becomes the A operand of a v_mfma_f32_32x32x16_f16, eight weights as f16:
//    (w & 0x000F000F) | 0x64006400 is the f16 pair (1024 + n0, 1024 + n4), minus 1032 it is (n0 - 8, n4 - 8), exact;
//    (w & 0x00F000F0) | 0x64006400 is (1024 + 16 n1, 1024 + 16 n5), minus 1152 it is 16 (n1 - 8), ...; w >> 8 gives
//    n2, n6, n3, n7 the same way; one packed multiply by the group's scale (or scale / 16) gives (n - 8) * scale
//    rounded to f16's 11 bits (the reference rounds it to bf16's 8, :311-312).  Twelve VALU operations per eight
//    weights and no conversion.  The eight values come out in the column order 0, 4, 1, 5, 2, 6, 3, 7; the
//    contraction order inside an MFMA is free, so the activations are stored in LDS in that order;
//  * the activations are the B operand: up to 32 tokens of the expert, converted bf16 -> f16 (exact for magnitudes
//    from 6.1e-5 to 65504; larger ones are clamped, smaller ones lose bits that a sum of 2048 or 7168 terms does not
//    see) and staged through LDS one run ahead, two buffers, rows padded by 16 bytes so that the operand reads are
//    free of bank conflicts; one workgroup barrier per run.
// Sums are fp32 (MFMA accumulators); the epilogue is the grouped GEMM's.
//
// MFMA's summation order is not documented and the weights carry three more bits than the reference's: this path
// is held to the 1e-2 bar like the other matrix-core paths, and is never used for the token-identity runs.
#include <atomic>
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_math.h"

namespace {

typedef _Float16 kx_h2 __attribute__((ext_vector_type(2)));
typedef _Float16 kx_h8 __attribute__((ext_vector_type(8)));
typedef float kx_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t kx_u32x4 __attribute__((ext_vector_type(4)));
// 16 bytes of a weight stream: non-temporal, they are used once
__device__ __forceinline__ uint4 mm_stream16(const uint4 *p) {
  const kx_u32x4 v = __builtin_nontemporal_load((const kx_u32x4 *)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}

constexpr int MM_RUN = 256;                   // columns per run: 128 bytes of a weight row
constexpr int MM_XPITCH = MM_RUN * 2 + 16;    // bytes per token row of a staged run of activations
constexpr int MM_XBUF = 32 * MM_XPITCH;
constexpr int MM_WAVES = 4;
constexpr int MM_WTILE = 32 * 128;            // bytes of a wave's staged weight run

struct MmArgs {
  const uint32_t *w0, *w1;   // packed i32 [E][N][K/8]
  const uint16_t *s0, *s1;   // bf16 scales [E][N][K/32]
  const uint16_t *x;         // bf16 activation rows of K
  uint16_t *out;             // bf16 [pairs][N]
  const int4 *work;          // {expert, first, last, _} per expert with work
  const int *pairs;          // pair ids sorted by expert
  int N, K, x_div;           // activation row = pair / x_div
  size_t expert_w, expert_s; // elements between experts (words; scales)
  int cnt_lo, cnt_hi;        // experts with fewer or more pairs are left to another launch
};

__device__ __forceinline__ uint32_t mm_and_or(uint32_t a, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(magic));
  return r;
}
// eight weights of a packed word as f16, (n - 8) * scale, in the column order 0, 4, 1, 5, 2, 6, 3, 7
__device__ __forceinline__ kx_h8 mm_dequant(uint32_t w, kx_h2 sc, kx_h2 sc16, uint32_t magic) {
  const kx_h2 off = {(_Float16)1032.0f, (_Float16)1032.0f}, off16 = {(_Float16)1152.0f, (_Float16)1152.0f};
  const uint32_t w8 = w >> 8;
  const kx_h2 a = (__builtin_bit_cast(kx_h2, mm_and_or(w, 0x000F000Fu, magic)) - off) * sc;       // n0, n4
  const kx_h2 b = (__builtin_bit_cast(kx_h2, mm_and_or(w, 0x00F000F0u, magic)) - off16) * sc16;   // n1, n5
  const kx_h2 c = (__builtin_bit_cast(kx_h2, mm_and_or(w8, 0x000F000Fu, magic)) - off) * sc;      // n2, n6
  const kx_h2 d = (__builtin_bit_cast(kx_h2, mm_and_or(w8, 0x00F000F0u, magic)) - off16) * sc16;  // n3, n7
  return __builtin_bit_cast(kx_h8, make_uint4(__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b),
                                              __builtin_bit_cast(uint32_t, c), __builtin_bit_cast(uint32_t, d)));
}
// bf16 pair (low, high halves of u) -> f16 pair, clamped to f16's range
__device__ __forceinline__ uint32_t mm_bf2_to_h2(uint32_t u) {
  const float lo = fminf(fmaxf(kx_bits_f32(u << 16), -65504.0f), 65504.0f);
  const float hi = fminf(fmaxf(kx_bits_f32(u & 0xffff0000u), -65504.0f), 65504.0f);
  const kx_h2 h = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, h);
}

// grid (N / 128, experts with work, passes of 32 tokens); 4 waves of 32 rows
template <bool DUAL>
__global__ void __launch_bounds__(MM_WAVES * 64, 2) i4mm_k(MmArgs a) {
  constexpr int MATS = DUAL ? 2 : 1;
  extern __shared__ __attribute__((aligned(16))) uint8_t mm_lds[];  // activations [2][32 tokens][MM_XPITCH], then the waves' weight tiles
  uint8_t *mm_x = mm_lds;
  const int4 rec = a.work[blockIdx.y];
  if (rec.x < 0) return;
  const int cnt = rec.z - rec.y;
  if (cnt < a.cnt_lo || cnt > a.cnt_hi) return;
  const int tok0 = rec.y + 32 * (int)blockIdx.z;
  if (tok0 >= rec.z) return;
  const int nt = min(32, rec.z - tok0);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int row0 = blockIdx.x * (MM_WAVES * 32) + wave * 32;
  const int K = a.K, nr = K / MM_RUN;
  const uint32_t magic = 0x64006400u;
  uint8_t *wt = mm_lds + 2 * MM_XBUF + wave * (MATS * MM_WTILE);  // this wave's tiles, one per matrix
  // loads of a run: instruction i takes rows 8 i .. + 7, eight lanes per row
  const int lrow = lane >> 3, lseg = lane & 7;
  const uint4 *wp[MATS];
  wp[0] = (const uint4 *)(a.w0 + (size_t)rec.x * a.expert_w + (size_t)(row0 + lrow) * (K / 8)) + lseg;
  if (DUAL) wp[1] = (const uint4 *)(a.w1 + (size_t)rec.x * a.expert_w + (size_t)(row0 + lrow) * (K / 8)) + lseg;
  const size_t wstride8 = (size_t)8 * (K / 8) / 4;  // uint4 between rows 8 apart
  // scales of the lane's row: groups 8 J + 4 h .. +3 of run J
  const uint2 *sp[MATS];
  sp[0] = (const uint2 *)(a.s0 + (size_t)rec.x * a.expert_s + (size_t)(row0 + r) * (K / 32)) + h;
  if (DUAL) sp[1] = (const uint2 *)(a.s1 + (size_t)rec.x * a.expert_s + (size_t)(row0 + r) * (K / 32)) + h;
  // activation staging: thread = (token, eighth): blocks of eight columns eighth, eighth + 8, ... of the run
  const int xt = threadIdx.x >> 3, xe = threadIdx.x & 7;
  const uint16_t *xrow = nullptr;
  if (xt < nt) xrow = a.x + (size_t)(a.pairs[tok0 + xt] / a.x_div) * K;
  uint4 xg[4];
  auto load_x = [&](int J) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      xg[i] = xrow ? *(const uint4 *)(xrow + J * MM_RUN + (xe + 8 * i) * 8) : make_uint4(0u, 0u, 0u, 0u);
  };
  auto store_x = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // columns 0..7 of the block as f16 pairs (0,1) (2,3) (4,5) (6,7), stored in the order 0, 4, 1, 5, 2, 6, 3, 7
      const uint32_t p01 = mm_bf2_to_h2(xg[i].x), p23 = mm_bf2_to_h2(xg[i].y), p45 = mm_bf2_to_h2(xg[i].z), p67 = mm_bf2_to_h2(xg[i].w);
      const uint4 o = make_uint4((p01 & 0xffffu) | (p45 << 16), (p01 >> 16) | (p45 & 0xffff0000u),
                                 (p23 & 0xffffu) | (p67 << 16), (p23 >> 16) | (p67 & 0xffff0000u));
      *(uint4 *)(mm_x + buf * MM_XBUF + xt * MM_XPITCH + (xe + 8 * i) * 16) = o;
    }
  };
  // a run's weights as loaded (line layout) and its scales
  uint4 ga[MATS][4], gb[MATS][4], gc[MATS][4];
  uint2 sa[MATS], sb[MATS], sc3[MATS];
  auto load_w = [&](uint4 (&gv)[MATS][4], uint2 (&sv)[MATS], int J) {
#pragma unroll
    for (int m = 0; m < MATS; ++m) {
#pragma unroll
      for (int i = 0; i < 4; ++i) gv[m][i] = mm_stream16(wp[m] + i * wstride8 + J * 8);
      sv[m] = sp[m][J * 2];
    }
  };
  kx_f32x16 acc[MATS];
#pragma unroll
  for (int m = 0; m < MATS; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;
  // run J from the registers gv: through the wave's LDS tile into the operand layout, then 16 products per matrix
  auto run = [&](const uint4 (&gv)[MATS][4], const uint2 (&sv)[MATS], int J) {
    if (J + 1 < nr) load_x(J + 1);
    uint4 w[MATS][4];
#pragma unroll
    for (int m = 0; m < MATS; ++m) {
#pragma unroll
      for (int i = 0; i < 4; ++i)  // row 8 i + lrow, piece lseg at slot lseg ^ (row % 8)
        *(uint4 *)(wt + m * MM_WTILE + (8 * i + lrow) * 128 + ((lseg ^ lrow) & 7) * 16) = gv[m][i];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int m = 0; m < MATS; ++m)
#pragma unroll
      for (int g = 0; g < 4; ++g) w[m][g] = *(const uint4 *)(wt + m * MM_WTILE + r * 128 + (((4 * h + g) ^ r) & 7) * 16);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const uint8_t *xb = mm_x + (J & 1) * MM_XBUF + r * MM_XPITCH + h * 256;  // token r, columns 128 h .. of the run
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      kx_h8 bx[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) bx[q] = *(const kx_h8 *)(xb + g * 64 + q * 16);
#pragma unroll
      for (int m = 0; m < MATS; ++m) {
        const uint32_t sd = (g & 2) ? sv[m].y : sv[m].x;
        const float sf = kx_bits_f32((g & 1) ? (sd & 0xffff0000u) : (sd << 16));
        const _Float16 s1 = (_Float16)sf, s16 = (_Float16)(sf * 0.0625f);
        const kx_h2 sc = {s1, s1}, sc16 = {s16, s16};
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(mm_dequant(w[m][g].x, sc, sc16, magic), bx[0], acc[m], 0, 0, 0);
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(mm_dequant(w[m][g].y, sc, sc16, magic), bx[1], acc[m], 0, 0, 0);
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(mm_dequant(w[m][g].z, sc, sc16, magic), bx[2], acc[m], 0, 0, 0);
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(mm_dequant(w[m][g].w, sc, sc16, magic), bx[3], acc[m], 0, 0, 0);
      }
    }
    if (J + 1 < nr) store_x((J + 1) & 1);
    __syncthreads();
  };

  // three register sets in rotation: two runs are on their way while one is multiplied
  load_w(ga, sa, 0);
  if (1 < nr) load_w(gb, sb, 1);
  load_x(0);
  store_x(0);
  __syncthreads();
  for (int J = 0; J < nr; J += 3) {
    if (J + 2 < nr) load_w(gc, sc3, J + 2);
    run(ga, sa, J);
    if (J + 1 < nr) {
      if (J + 3 < nr) load_w(ga, sa, J + 3);
      run(gb, sb, J + 1);
    }
    if (J + 2 < nr) {
      if (J + 4 < nr) load_w(gb, sb, J + 4);
      run(gc, sc3, J + 2);
    }
  }
  // D[i][j]: i = weight row 8 (v / 4) + 4 h + v % 4 of the wave's 32, j = token r
  if (r < nt) {
    const int pr = a.pairs[tok0 + r];
    uint16_t *o = a.out + (size_t)pr * a.N + row0 + 4 * h;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint16_t v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float y = acc[0][4 * q + e];
        if (DUAL) y = kx_swiglu(kx_bfround(y), kx_bfround(acc[MATS - 1][4 * q + e]));
        v[e] = kx_bf16_rne(y);
      }
      *(uint2 *)(o + 8 * q) = make_uint2((uint32_t)v[0] | ((uint32_t)v[1] << 16), (uint32_t)v[2] | ((uint32_t)v[3] << 16));
    }
  }
}

}  // namespace

// The experts of the work list with cnt_lo .. cnt_hi pairs (at most 32 per pass; more take further passes):
// out[pair][N] = W[expert] x[pair / x_div], or, with two matrices, swiglu(W0 x, W1 x).  *done = false, nothing
// launched, when the shape is not the kernel's.
int kx_i4mm_launch(bool dual, const uint32_t *w0, const uint16_t *s0, const uint32_t *w1, const uint16_t *s1, const uint16_t *x,
                   uint16_t *out, const int4 *work, const int *pairs, int n_slots, int N, int K, int x_div, size_t expert_w,
                   size_t expert_s, int cnt_lo, int cnt_hi, int passes, bool *done, hipStream_t st) {
  *done = false;
  if (!(N > 0 && N % (MM_WAVES * 32) == 0 && K > 0 && K % MM_RUN == 0 && n_slots > 0 && passes > 0 && x_div > 0)) return KX_OK;
  MmArgs a;
  a.w0 = w0; a.w1 = w1; a.s0 = s0; a.s1 = s1; a.x = x; a.out = out; a.work = work; a.pairs = pairs;
  a.N = N; a.K = K; a.x_div = x_div; a.expert_w = expert_w; a.expert_s = expert_s; a.cnt_lo = cnt_lo; a.cnt_hi = cnt_hi;
  const size_t lds = 2 * MM_XBUF + (size_t)MM_WAVES * (dual ? 2 : 1) * MM_WTILE;
  static std::atomic<bool> attr_set{false};
  if (!attr_set) {
    KX_HIP(hipFuncSetAttribute((const void *)i4mm_k<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * MM_XBUF + MM_WAVES * 2 * MM_WTILE));
    KX_HIP(hipFuncSetAttribute((const void *)i4mm_k<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * MM_XBUF + MM_WAVES * MM_WTILE));
    attr_set = true;
  }
  const dim3 g(N / (MM_WAVES * 32), n_slots, passes), b(MM_WAVES * 64);
  if (dual) hipLaunchKernelGGL(i4mm_k<true>, g, b, lds, st, a);
  else hipLaunchKernelGGL(i4mm_k<false>, g, b, lds, st, a);
  KX_LAUNCH_CHECK();
  *done = true;
  return KX_OK;
}
