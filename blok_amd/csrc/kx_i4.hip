// kx_i4.hip -- compressed-tensors INT4 (pack_quantized, group 32, bf16 scales):
// unpack, dequant and the fused W4A16 GEMV used by routed-expert decode.
//
// Reference: matvec_i4_bf16_scale_k, src/kimi_exec.cu:300-323 (one 256-thread
// block per output row, one thread per 32-weight group, per-nibble shift /
// mask / convert / round / FMA).  This file keeps the data format and the
// result within bf16 tolerance, and replaces the schedule:
//
//  * a lane owns one 32-weight group = one 128-bit load of packed words;
//    a half-wave (32 lanes) covers a 1024-column slice of a row with one
//    512-byte contiguous read, the other half-wave takes the next row;
//  * the activations of the lane's group stay in registers as f32 across all
//    rows of the work item (half of them pre-divided by 16, see below);
//  * nibbles are turned into f16 values without shifts where possible:
//    (w & 0x000F000F) | 0x64006400 is the f16 pair (1024+n0, 1024+n4) and
//    (w & 0x00F000F0) | 0x64006400 is (1024+16*n1, 1024+16*n5); w >> 8 gives
//    n2,n6,n3,n7 the same way.  v_fma_mix_f32 multiplies an f16 operand into
//    an f32 accumulator with a single rounding, so a word costs 1 shift,
//    4 and-or and 8 fma;
//  * the offsets (1024, and the -8 of q = n - 8) are folded into the start
//    value of the accumulator: acc0 = -sum_k x'_k * c_k with c = 1032 for
//    nibbles 0,2,4,6 and 1152 for nibbles 1,3,5,7 (x' = x/16 there);
//  * the group scale is applied once per group: part = scale * acc;
//  * reductions: xor-butterfly over the 32 lanes of the half-wave
//    (16,8,4,2,1), then a sequential sum over the 1024-column slices.
//
// All arithmetic is IEEE binary32 (fma, mul, add), so a scalar host program
// that follows the same order reproduces the result bit for bit.
#include "kx_common.h"
#include "kx_math.h"

namespace {

typedef _Float16 kx_h2 __attribute__((ext_vector_type(2)));
typedef unsigned int kx_u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(magic));
  return r;
}

// streaming 128-bit load: the weights are read once, keep them out of the way
__device__ __forceinline__ uint4 ld_stream(const uint32_t *p) {
  kx_u32x4 v = __builtin_nontemporal_load((const kx_u32x4 *)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}

// ---- elementwise: unpack and dequant -----------------------------------------
__global__ void i4_unpack_k(const uint32_t *__restrict__ packed, int8_t *__restrict__ q, size_t n_words) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_words) return;
  uint32_t w = packed[i];
  uint32_t lo = 0, hi = 0;
  for (int j = 0; j < 4; ++j) {
    lo |= (uint32_t)(uint8_t)(int8_t)((int)((w >> (4 * j)) & 0xfu) - 8) << (8 * j);
    hi |= (uint32_t)(uint8_t)(int8_t)((int)((w >> (4 * (j + 4))) & 0xfu) - 8) << (8 * j);
  }
  ((uint2 *)q)[i] = make_uint2(lo, hi);
}

__global__ void i4_dequant_k(const uint32_t *__restrict__ packed, const uint16_t *__restrict__ scale,
                             uint16_t *__restrict__ w_out, size_t n_words) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // word index; 4 words per group
  if (i >= n_words) return;
  uint32_t w = packed[i];
  float sc = kx_bf16_f32(scale[i >> 2]);
  uint32_t o[4];
  for (int j = 0; j < 4; ++j) {
    int q0 = (int)((w >> (8 * j)) & 0xfu) - 8, q1 = (int)((w >> (8 * j + 4)) & 0xfu) - 8;
    o[j] = (uint32_t)kx_bf16_rne((float)q0 * sc) | ((uint32_t)kx_bf16_rne((float)q1 * sc) << 16);
  }
  ((uint4 *)w_out)[i] = make_uint4(o[0], o[1], o[2], o[3]);
}

// ---- fused GEMV -----------------------------------------------------------------
// activations of one group in chain order; entries 2,3,6,7 of each 8 hold x/16
struct XGroup {
  float v[32];
  float neg_c;  // -(sum of offsets), the start value of every chain
};

__device__ __forceinline__ float bf_lo(uint32_t u) { return kx_bits_f32(u << 16); }
__device__ __forceinline__ float bf_hi(uint32_t u) { return kx_bits_f32(u & 0xffff0000u); }

__device__ __forceinline__ void load_xgroup(XGroup &g, const uint16_t *x /* 32 bf16, 64 B aligned */) {
  const uint4 *p = (const uint4 *)x;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    uint4 u = p[w];  // x[8w .. 8w+7]
    g.v[w * 8 + 0] = bf_lo(u.x);             // k = 8w+0
    g.v[w * 8 + 1] = bf_lo(u.z);             // k = 8w+4
    g.v[w * 8 + 2] = bf_hi(u.x) * 0.0625f;   // k = 8w+1
    g.v[w * 8 + 3] = bf_hi(u.z) * 0.0625f;   // k = 8w+5
    g.v[w * 8 + 4] = bf_lo(u.y);             // k = 8w+2
    g.v[w * 8 + 5] = bf_lo(u.w);             // k = 8w+6
    g.v[w * 8 + 6] = bf_hi(u.y) * 0.0625f;   // k = 8w+3
    g.v[w * 8 + 7] = bf_hi(u.w) * 0.0625f;   // k = 8w+7
  }
  float c = 0.0f;
#pragma unroll
  for (int i = 0; i < 32; ++i) c = __builtin_fmaf(g.v[i], ((i & 2) ? 1152.0f : 1032.0f), c);
  g.neg_c = -c;
}

struct I4Dec {  // the eight f16 pairs of one 128-bit load... four words, four pairs each
  kx_h2 a[16];
};

__device__ __forceinline__ void decode_words(I4Dec &d, uint4 v, uint32_t magic) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    uint32_t w8 = w[p] >> 8;
    d.a[p * 4 + 0] = __builtin_bit_cast(kx_h2, and_or(w[p], 0x000F000Fu, magic));
    d.a[p * 4 + 1] = __builtin_bit_cast(kx_h2, and_or(w[p], 0x00F000F0u, magic));
    d.a[p * 4 + 2] = __builtin_bit_cast(kx_h2, and_or(w8, 0x000F000Fu, magic));
    d.a[p * 4 + 3] = __builtin_bit_cast(kx_h2, and_or(w8, 0x00F000F0u, magic));
  }
}

__device__ __forceinline__ float group_dot(const I4Dec &d, const XGroup &g) {
  float acc = g.neg_c;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    acc = __builtin_fmaf((float)d.a[i].x, g.v[2 * i], acc);
    acc = __builtin_fmaf((float)d.a[i].y, g.v[2 * i + 1], acc);
  }
  return acc;
}

__device__ __forceinline__ float half_wave_sum(float v) {
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 8);
  v += __shfl_xor(v, 4);
  v += __shfl_xor(v, 2);
  v += __shfl_xor(v, 1);
  return v;
}

struct I4Args {
  const uint32_t *packed0;
  const uint16_t *scale0;
  const uint32_t *packed1;  // DUAL only
  const uint16_t *scale1;
  const uint16_t *x;  // bf16 rows of `cols`
  uint16_t *out;      // bf16 rows of `rows`, indexed by pair
  const int *active;  // expert ids with work; nullptr: one matrix, pairs 0..n_pairs-1
  const int *n_active;
  const int *offsets;  // [E+1] exclusive offsets into pairs
  const int *pairs;    // pair ids sorted by expert
  int n_pairs;         // used when active == nullptr
  int rows, cols;
  int x_div;  // activation row = pair / x_div
  int ks, rs;  // 1024-column slices, row sets; ks*rs waves per workgroup
  size_t expert_words, expert_scales;
};

// RI rows per half-wave per item, TT tokens per pass
template <bool DUAL, int RI, int TT>
__global__ void __launch_bounds__(1024) i4_gemv_k(I4Args a) {
  extern __shared__ float lds[];  // [mats][RT][TT][ks] partials, then scale tiles
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l = lane & 31, h = lane >> 5;
  const int s = wave % a.ks, rset = wave / a.ks;
  const int RT = a.rs * 2 * RI;  // rows per item
  const int MATS = DUAL ? 2 : 1;
  const int groups = a.cols >> 5;
  float *part = lds;
  uint16_t *sc_lds = (uint16_t *)(lds + MATS * RT * TT * a.ks);  // [mats][RT][groups]
  const int tiles = (a.rows + RT - 1) / RT;
  const int n_active = a.active ? *a.n_active : 1;
  const int n_items = n_active * tiles;
  uint32_t magic;
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));

  for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
    const int ai = item / tiles, tile = item - ai * tiles;
    const int e = a.active ? a.active[ai] : 0;
    const int p_begin = a.active ? a.offsets[e] : 0;
    const int p_end = a.active ? a.offsets[e + 1] : a.n_pairs;
    const int r0 = tile * RT;
    const uint32_t *pk[2] = {a.packed0 + (size_t)e * a.expert_words,
                             DUAL ? a.packed1 + (size_t)e * a.expert_words : nullptr};
    const uint16_t *scg[2] = {a.scale0 + (size_t)e * a.expert_scales,
                              DUAL ? a.scale1 + (size_t)e * a.expert_scales : nullptr};

    // issue the weight loads of this item first
    uint4 wv[MATS][RI];
    int rows_i[RI];
#pragma unroll
    for (int i = 0; i < RI; ++i) {
      int row = r0 + (rset * RI + i) * 2 + h;
      rows_i[i] = row;
      int row_c = row < a.rows ? row : a.rows - 1;
#pragma unroll
      for (int m = 0; m < MATS; ++m)
        wv[m][i] = ld_stream(pk[m] + (size_t)row_c * (a.cols >> 3) + (size_t)(s * 32 + l) * 4);
    }
    // stage the scale rows of the tile in LDS (contiguous in memory)
    {
      const int rows_here = min(RT, a.rows - r0);
      const int n16 = rows_here * groups / 8;  // uint4 chunks (groups is a multiple of 32)
      for (int m = 0; m < MATS; ++m) {
        const uint4 *src = (const uint4 *)(scg[m] + (size_t)r0 * groups);
        uint4 *dst = (uint4 *)(sc_lds + (size_t)m * RT * groups);
        for (int i = threadIdx.x; i < n16; i += blockDim.x) dst[i] = src[i];
      }
    }
    __syncthreads();
    float scf[MATS][RI];
#pragma unroll
    for (int i = 0; i < RI; ++i)
#pragma unroll
      for (int m = 0; m < MATS; ++m) {
        int rt = min(rows_i[i], a.rows - 1) - r0;
        scf[m][i] = kx_bf16_f32(sc_lds[((size_t)m * RT + rt) * groups + s * 32 + l]);
      }

    for (int pc = p_begin; pc < p_end; pc += TT) {
      XGroup xg[TT];
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        int pi = min(pc + t, p_end - 1);
        int pair = a.active ? a.pairs[pi] : pi;
        load_xgroup(xg[t], a.x + (size_t)(pair / a.x_div) * a.cols + (size_t)(s * 32 + l) * 32);
      }
#pragma unroll
      for (int i = 0; i < RI; ++i)
#pragma unroll
        for (int m = 0; m < MATS; ++m) {
          I4Dec dec;
          decode_words(dec, wv[m][i], magic);
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            float v = scf[m][i] * group_dot(dec, xg[t]);
            v = half_wave_sum(v);
            if (l == 0) part[((m * RT + (rset * RI + i) * 2 + h) * TT + t) * a.ks + s] = v;
          }
        }
      __syncthreads();
      // sequential sum over the slices, rounding and epilogue
      for (int idx = threadIdx.x; idx < RT * TT; idx += blockDim.x) {
        int rt = idx % RT, t = idx / RT;
        int row = r0 + rt;
        if (row < a.rows && pc + t < p_end) {
          int pair = a.active ? a.pairs[pc + t] : pc + t;
          const float *p0 = part + ((0 * RT + rt) * TT + t) * a.ks;
          float y0 = p0[0];
          for (int q = 1; q < a.ks; ++q) y0 += p0[q];
          float res;
          if (DUAL) {
            const float *p1 = part + ((1 * RT + rt) * TT + t) * a.ks;
            float y1 = p1[0];
            for (int q = 1; q < a.ks; ++q) y1 += p1[q];
            res = kx_swiglu(kx_bfround(y0), kx_bfround(y1));
          } else {
            res = y0;
          }
          a.out[(size_t)pair * a.rows + row] = kx_bf16_rne(res);
        }
      }
      __syncthreads();
    }
  }
}

struct I4Launch {
  int ks, rs, threads, rt;
  size_t lds;
};

template <int RI>
int plan(int cols, int rows, int mats, int tt, I4Launch &pl) {
  KX_REQUIRE(cols > 0 && cols % 1024 == 0, "kx_i4: cols=%d must be a positive multiple of 1024", cols);
  KX_REQUIRE(rows > 0, "kx_i4: rows=%d must be positive", rows);
  pl.ks = cols / 1024;
  KX_REQUIRE(pl.ks <= 16, "kx_i4: cols=%d exceeds 16384", cols);
  pl.rs = pl.ks >= 7 ? 1 : (8 / pl.ks);
  pl.threads = pl.ks * pl.rs * 64;
  pl.rt = pl.rs * 2 * RI;
  pl.lds = (size_t)mats * pl.rt * tt * pl.ks * sizeof(float) + (size_t)mats * pl.rt * (cols / 32) * 2;
  return KX_OK;
}

}  // namespace

// rows per half-wave per item
#define KX_I4_RI 4

// Launches the fused gate/up (DUAL) or single-matrix GEMV over a bucketed pair
// list.  max_pairs_per_expert picks the tokens-per-pass variant.
int kx_i4_launch(bool dual, const uint32_t *packed0, const uint16_t *scale0, const uint32_t *packed1,
                 const uint16_t *scale1, const uint16_t *x, uint16_t *out, const int *active,
                 const int *n_active, const int *offsets, const int *pairs, int n_pairs, int rows,
                 int cols, int x_div, size_t expert_words, size_t expert_scales, int tt, int grid,
                 hipStream_t st) {
  I4Launch pl;
  int rc = plan<KX_I4_RI>(cols, rows, dual ? 2 : 1, tt, pl);
  if (rc) return rc;
  I4Args a;
  a.packed0 = packed0; a.scale0 = scale0; a.packed1 = packed1; a.scale1 = scale1;
  a.x = x; a.out = out; a.active = active; a.n_active = n_active; a.offsets = offsets; a.pairs = pairs;
  a.n_pairs = n_pairs; a.rows = rows; a.cols = cols; a.x_div = x_div; a.ks = pl.ks; a.rs = pl.rs;
  a.expert_words = expert_words; a.expert_scales = expert_scales;
  dim3 g(grid), b(pl.threads);
  if (dual) {
    if (tt == 1) hipLaunchKernelGGL((i4_gemv_k<true, KX_I4_RI, 1>), g, b, pl.lds, st, a);
    else if (tt == 2) hipLaunchKernelGGL((i4_gemv_k<true, KX_I4_RI, 2>), g, b, pl.lds, st, a);
    else hipLaunchKernelGGL((i4_gemv_k<true, KX_I4_RI, 4>), g, b, pl.lds, st, a);
  } else {
    if (tt == 1) hipLaunchKernelGGL((i4_gemv_k<false, KX_I4_RI, 1>), g, b, pl.lds, st, a);
    else if (tt == 2) hipLaunchKernelGGL((i4_gemv_k<false, KX_I4_RI, 2>), g, b, pl.lds, st, a);
    else hipLaunchKernelGGL((i4_gemv_k<false, KX_I4_RI, 4>), g, b, pl.lds, st, a);
  }
  KX_LAUNCH_CHECK();
  return KX_OK;
}

extern "C" int kx_i4_unpack(const void *d_packed, void *d_q, int32_t rows, int32_t cols, void *stream) {
  KX_REQUIRE(d_packed && d_q, "kx_i4_unpack: null pointer");
  KX_REQUIRE(rows > 0 && cols > 0 && cols % 8 == 0, "kx_i4_unpack: rows=%d cols=%d (cols must be a multiple of 8)", rows, cols);
  size_t n_words = (size_t)rows * (cols / 8);
  hipLaunchKernelGGL(i4_unpack_k, dim3((unsigned)((n_words + 255) / 256)), dim3(256), 0, kx_stream(stream),
                     (const uint32_t *)d_packed, (int8_t *)d_q, n_words);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

extern "C" int kx_i4_dequant(const void *d_packed, const void *d_scale, void *d_w, int32_t rows, int32_t cols,
                             void *stream) {
  KX_REQUIRE(d_packed && d_scale && d_w, "kx_i4_dequant: null pointer");
  KX_REQUIRE(rows > 0 && cols > 0 && cols % 32 == 0, "kx_i4_dequant: rows=%d cols=%d (cols must be a multiple of 32)", rows, cols);
  size_t n_words = (size_t)rows * (cols / 8);
  hipLaunchKernelGGL(i4_dequant_k, dim3((unsigned)((n_words + 255) / 256)), dim3(256), 0, kx_stream(stream),
                     (const uint32_t *)d_packed, (const uint16_t *)d_scale, (uint16_t *)d_w, n_words);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

extern "C" int kx_i4_gemv(const void *d_packed, const void *d_scale, const void *d_x, void *d_y, int32_t rows,
                          int32_t cols, int32_t tokens, void *stream) {
  KX_REQUIRE(d_packed && d_scale && d_x && d_y, "kx_i4_gemv: null pointer");
  KX_REQUIRE(tokens > 0, "kx_i4_gemv: tokens=%d must be positive", tokens);
  int tt = tokens >= 4 ? 4 : tokens >= 2 ? 2 : 1;
  I4Launch pl;
  int rc = plan<KX_I4_RI>(cols, rows, 1, tt, pl);
  if (rc) return rc;
  int tiles = kx_cdiv(rows, pl.rt);
  int grid = tiles < 1024 ? tiles : 1024;
  return kx_i4_launch(false, (const uint32_t *)d_packed, (const uint16_t *)d_scale, nullptr, nullptr,
                      (const uint16_t *)d_x, (uint16_t *)d_y, nullptr, nullptr, nullptr, nullptr, tokens, rows,
                      cols, 1, 0, 0, tt, grid, kx_stream(stream));
}
