// kx_mla.hip -- MLA decode attention on the absorbed latent KV cache, with the
// RMSNorm / RoPE steps that sit on its path.
//
// Reference: the attention half of run(), src/kimi_exec.cu:812-827 -- q_a/q_b and
// kv_a/kv_b projections, rope_k (:346-357) with the YaRN frequencies (:325-344),
// an expanded fp32 K/V cache on NVMe (:192-238) and tiled_attention (:692-716),
// a three-pass softmax that streams every K tile three times.  Here the cache
// holds what kv_a produced: per position the RMS-normed 512-d latent and the
// rotated 64-d rope key (bf16, 1152 B instead of 81920 B), and the kv_b
// projection is absorbed into the query and the output:
//   q_lat[h] = bf(W_UK[h]^T q_nope[h])            (W_UK[h] = kv_b rows h*256 .. +127)
//   s[t,h]   = bf(bf(q_lat[h].c_t + q_rope[h].k_rope_t) * rsqrt(192) * mscale^2)
//   o_lat[h] = softmax(s)[t] . c_t ;  o[h] = bf(W_UV[h] o_lat[h])   (rows h*256+128 ..)
// One pass over the cache with an online softmax; the sequence is cut into spans
// of span_tiles 64-position tiles that run in parallel and are merged afterwards.
// Two kernels compute the span partials: mla_partial_k (fp32 VALU, the fixed summation
// order below) and, for long contexts, mla_partial_mfma_k on the matrix cores.
//
// Summation order of the VALU path (fixed; span_tiles depends on the sequence length only):
//   score      one fma chain over the 576 cache columns, ascending
//   tile       m = max s; p = exp(s - M'); z = xor-butterfly(64) of p;
//              running: M' = max(M, m), a = exp(M - M'), Z = fma(Z, a, z),
//              O[c] = (O[c] * a) then fma chain over the tile's positions of bf(p) * c_t[c]
//   merge      M = max M_j; w_j = exp(M_j - M); Z = fma(Z_j, w_j, Z), O = fma(O_j, w_j, O)
//              over spans ascending; o_lat = bf(O / Z)
//   q_lat      eight chains over d = j, j+8, ... then ((0+1)+(2+3))+((4+5)+(6+7))
#include <math.h>
#include <atomic>
#include <type_traits>
#include "kx_attn_parts.h"
#include "kx_common.h"
#include "kx_lds_copy.h"
#include "kx_dense.h"
#include "kx_math.h"
#include "kx_mla.h"
#include "kx_wave.h"

// ---- host: YaRN frequencies, rope table, score scale ---------------------------------
static float yarn_correction_dim(const kx_config *c, float rotations, float dim) {  // :325-327
  volatile float two_pi = 2.0f * 3.14159265358979323846f;
  return dim * logf(c->yarn_orig_ctx / (rotations * two_pi)) / (2.0f * logf(c->rope_theta));
}
static float yarn_inv_freq(const kx_config *c, int pair) {  // :334-344
  const float dim = (float)c->qk_rope;
  const float freq_extra = powf(c->rope_theta, -2.0f * (float)pair / dim);
  const float freq_inter = freq_extra / c->yarn_factor;
  float low = floorf(yarn_correction_dim(c, c->yarn_beta_fast, dim));
  float high = ceilf(yarn_correction_dim(c, c->yarn_beta_slow, dim));
  low = fmaxf(low, 0.0f);
  high = fminf(high, dim - 1.0f);
  if (low == high) high += 0.001f;  // :330
  const float ramp = fminf(1.0f, fmaxf(0.0f, ((float)pair - low) / (high - low)));
  const float mask = 1.0f - ramp;
  return freq_inter * (1.0f - mask) + freq_extra * mask;
}

extern "C" int kx_rope_table(const kx_config *cfg, int32_t pos0, int32_t n, uint16_t *h_out) {
  KX_REQUIRE(cfg && h_out, "kx_rope_table: null argument");
  KX_REQUIRE(cfg->qk_rope > 0 && cfg->qk_rope % 2 == 0 && n >= 0 && pos0 >= 0, "kx_rope_table: bad shape");
  const int half = cfg->qk_rope / 2;
  for (int p = 0; p < half; ++p) {
    const float freq = yarn_inv_freq(cfg, p);
    for (int i = 0; i < n; ++i) {
      const float ang = (float)(pos0 + i) * freq;  // :351, int * float
      h_out[(size_t)i * cfg->qk_rope + p] = kx_bf16_rne(cosf(ang));
      h_out[(size_t)i * cfg->qk_rope + half + p] = kx_bf16_rne(sinf(ang));
    }
  }
  return KX_OK;
}

extern "C" int kx_softmax_scale(const kx_config *cfg, float *rs, float *mscale) {
  KX_REQUIRE(cfg && rs && mscale, "kx_softmax_scale: null argument");
  *rs = kx_rsqrtf((float)(cfg->qk_nope + cfg->qk_rope));
  *mscale = 0.1f * cfg->yarn_mscale_all_dim * logf(cfg->yarn_factor) + 1.0f;  // :428
  return KX_OK;
}


int kx_mla_span_tiles(int seq) {
  int tiles = (seq + 63) / 64, st = 1;
  while (tiles > 64 * st) st *= 2;
  return st;
}

// The matrix-core kernel is not tied to that partition (it is held to a tolerance, not to the oracle's sums): few
// sequences get more, shorter spans so that sequences x spans fills the chip -- up to 256 spans, merged 64 at a time.
// Beyond 32 entries (the launches of a prefill step) the entries alone fill the chip and every span costs a row of
// partials that is written and read back: down to 4 spans.
static int mla_compute_units() {  // of the current device, asked once
  static std::atomic<int> cus{0};
  int v = cus.load();
  if (!v) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cus = v;
  }
  return v;
}
static int mfma_span_cap(int batch) {
  if (batch > 32) return 2048 / batch < 4 ? 4 : 2048 / batch;
  const int want = 1024 / (batch > 0 ? batch : 1);
  return want > 256 ? 256 : want < 64 ? 64 : want;
}
static int mfma_span_tiles(int seq, int batch) {
  const int tiles = (seq + 63) / 64, cap = mfma_span_cap(batch);
  int st = 1;
  while (tiles > cap * st) st *= 2;
  if (batch > 32) return st;
  // Up to 32 sequences: longer spans than the cap asks for, where that is cheaper.  A span costs a row of partials
  // per head (2 KB written, read back and merged), and workgroups come in rounds of one per CU, so the time of a
  // partition goes like rounds x tiles per span + c x spans, in units of a tile's time, with c = 0.017 x sequences
  // (fitted: 16 sequences of 131072 positions, 64 spans against 16).  Measured with this choice against the cap
  // alone, ms: 16 x 131072: 0.559 against 0.616; 16 x 32768: 0.154 against 0.239; 16 x 4096: 0.040 against 0.102;
  // 8 x 32768: 0.081 against 0.158; 32 x 4096: 0.056 against 0.222.
  const int cus = mla_compute_units();
  auto cost = [&](int t) {
    const int spans = (tiles + t - 1) / t;
    const long rounds = ((long)batch * spans + cus - 1) / cus;
    return (double)rounds * t + 0.017 * batch * spans;
  };
  int best = st;
  for (int t = st * 2; t <= tiles * 2 && t <= 4096; t *= 2)
    if (cost(t) < cost(best)) best = t;
  return best;
}

namespace {

using kxg::bf_hi;
using kxg::bf_lo;
using kxg::unpack8;
using namespace kxa;

// q_abs[t][h] = (bf(W_UK[h]^T q_nope[h]) | rope(q_rope[h])) as f32.  A workgroup of 128 threads takes
// 128 latent columns of one head: thread (chain, cl) = (tid / 16, tid % 16) runs the fma chain over
// d = chain, chain+8, ... for columns 8 cl .. 8 cl + 7; the 8 chains are then summed pairwise.
// Grid (heads * ceil(kv_rank / 128) + 1, T): the extra workgroup finishes the token's kv_a output and
// writes its cache row.
// TB tokens per workgroup (blockIdx.y = block of TB tokens): a weight is loaded once for all of them, and each token's
// sums are those of one token alone.  One token per workgroup reads the head's W_UK from L2 once per token, which
// bounds the kernel from about 8 tokens on.
template <int TB>
__global__ void __launch_bounds__(128) q_absorb_k(QAbsArgs a, int tokens) {
  __shared__ float part[TB][8][128];
  __shared__ float ws[4];
  const int t0 = blockIdx.y * TB;
  const int nope = a.nope, rope = a.rope, kv_rank = a.kv_rank;
  const int qk = nope + rope, kva = kv_rank + rope;
  const int cq_n = (kv_rank + 127) >> 7;
  if ((int)blockIdx.x == a.heads * cq_n) {
    if (a.cache)
      for (int t = t0; t < min(t0 + TB, tokens); ++t) {
        const int sb = a.seqs ? t % a.seqs : t, i = a.seqs ? t / a.seqs : 0;
        kv_finish_block(a.kva + (size_t)t * a.kva_stride, a.w_kv_ln, a.rope_row + (size_t)i * rope,
                        a.cache + (size_t)sb * a.seq_stride + (size_t)(a.pos + i) * kva, kv_rank, rope, a.eps, ws);
        __syncthreads();  // ws is reused by the next token
      }
    return;
  }
  const int h = blockIdx.x / cq_n, cq = blockIdx.x - h * cq_n;
  const int cl = threadIdx.x & 15, chain = threadIdx.x >> 4;
  const uint16_t *qh[TB];
#pragma unroll
  for (int i = 0; i < TB; ++i) qh[i] = a.q + ((size_t)min(t0 + i, tokens - 1) * a.heads + h) * qk;
  const uint16_t *wuk = a.kvb + (size_t)h * (nope + a.v_head) * kv_rank;
  const int c0 = cq * 128 + cl * 8;
  if (c0 < kv_rank) {
    float acc[TB][8];
#pragma unroll
    for (int i = 0; i < TB; ++i)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[i][e] = 0.0f;
#pragma unroll TB == 1 ? 16 : 4
    for (int d = chain; d < nope; d += 8) {
      float wf[8];
      unpack8(wf, *(const uint4 *)(wuk + (size_t)d * kv_rank + c0));
#pragma unroll
      for (int i = 0; i < TB; ++i) {
        const float qd = kx_bf16_f32(qh[i][d]);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[i][e] = __builtin_fmaf(wf[e], qd, acc[i][e]);
      }
    }
#pragma unroll
    for (int i = 0; i < TB; ++i)
#pragma unroll
      for (int e = 0; e < 8; ++e) part[i][chain][cl * 8 + e] = acc[i][e];
  }
  __syncthreads();
  const int half = rope >> 1;
#pragma unroll
  for (int i = 0; i < TB; ++i) {
    if (t0 + i >= tokens) break;
    float *out = a.qabs + ((size_t)(t0 + i) * a.heads + h) * kva;
    const int c = threadIdx.x;
    if (cq * 128 + c < kv_rank) {
      const float s = ((part[i][0][c] + part[i][1][c]) + (part[i][2][c] + part[i][3][c])) + ((part[i][4][c] + part[i][5][c]) + (part[i][6][c] + part[i][7][c]));
      out[cq * 128 + c] = kx_bfround(s);
    }
    if (cq == 0 && (int)threadIdx.x < half) {
      const int p = threadIdx.x;
      const uint16_t *rr = a.rope_row + (size_t)(a.seqs ? (t0 + i) / a.seqs : 0) * rope;
      float lo, hi;
      rope_pair(kx_bf16_f32(qh[i][nope + 2 * p]), kx_bf16_f32(qh[i][nope + 2 * p + 1]), kx_bf16_f32(rr[p]),
                kx_bf16_f32(rr[half + p]), lo, hi);
      out[kv_rank + p] = lo;
      out[kv_rank + half + p] = hi;
    }
  }
}

struct MlaArgs {
  const uint16_t *cache;  // bf16 [B][seq_stride/kva positions][kva]
  const float *qabs;      // f32 [B][heads][kva]
  float *pm, *pz, *po;    // partials [B][spans][heads], same, [B][spans][heads][kv_rank]
  int heads, seq, span_tiles, spans;
  int seqs;               // 0: grid index z is sequence z, which attends `seq` positions.  n > 0 (a prefill step of
                          // several positions of n sequences): z = i * n + b is position i of sequence b; it reads
                          // cache block b and attends seq - (grid z / n - 1) + i positions, the last position all `seq`
  size_t seq_stride;      // elements between sequences in the cache
  float rs, mscale;
};

// kv_rank 512, rope 64 (the Kimi-K2 latent layout).  HG heads per wave, 4 waves per workgroup.
// grid (spans, heads / (4*HG), B).  The 64 cache rows of a tile are staged in LDS once per
// workgroup with coalesced 16-byte loads (row pitch 1168 B, so that both the row-per-lane reads
// of the score pass and the column-per-lane reads of the PV pass are free of bank conflicts).
constexpr int MLA_R = 512, MLA_KVA = 576, MLA_PITCH = 584;  // bf16 elements; 1168 B per staged row
constexpr int MLA_PITCH_F = 580;  // F32: floats per staged row (2320 B: 580 mod 32 = 4, so eight rows' 16-byte reads cover all banks)

// W waves per workgroup, HG heads per wave.  The waves of a workgroup share the staged tile; with W = 6 .. 8 (HG = 1)
// the last workgroup of a span may hold waves past the last head: they stage and keep the barriers, and compute the
// last head again without storing it.
// F32 (launches of at most one workgroup per CU, which then has the LDS for it): the tile is staged as floats, the
// bf16 -> f32 conversion done once by the threads that stage instead of by every wave on every read: half of a
// wave's VALU work in both passes is that conversion, and the SIMDs that hold two waves are what the launch waits
// for.  The values and the order of the sums are the same.
template <int HG, int W = 4, bool F32 = false>
__global__ void __launch_bounds__(W * 64) mla_partial_k(MlaArgs a) {
  constexpr int R = MLA_R, KVA = MLA_KVA, PITCH = MLA_PITCH, PITCH_F = MLA_PITCH_F;
  extern __shared__ __attribute__((aligned(16))) uint16_t tile_lds[];  // [64][PITCH] bf16 or [64][PITCH_F] floats, then p [W][HG][64] floats
  float *tile_f = (float *)tile_lds;
  float(*p_lds)[HG][64] = F32 ? (float(*)[HG][64])(tile_f + 64 * PITCH_F) : (float(*)[HG][64])(tile_lds + 64 * PITCH);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: q is then read through the scalar path
  const int span = blockIdx.x, b = blockIdx.z;
  const int h_own = (blockIdx.y * W + wave) * HG;
  const bool h_valid = h_own < a.heads;
  const int h0 = h_valid ? h_own : a.heads - HG;
  const int seq = a.seqs ? a.seq - (int)(gridDim.z / a.seqs) + 1 + b / a.seqs : a.seq;
  const uint16_t *cache = a.cache + (size_t)(a.seqs ? b % a.seqs : b) * a.seq_stride;
  const float *q = a.qabs + ((size_t)b * a.heads + h0) * KVA;
  const int tiles = (seq + 63) >> 6;  // a span past them leaves M = -inf, Z = 0, O = 0, which the merge weighs with 0
  const int tile_end = min(tiles, (span + 1) * a.span_tiles);
  // the lane's 8 latent columns in the PV pass: contiguous over the bf16 tile; two groups of four, 256 apart, over the
  // float tile, so that a wave's reads of a row are two runs of 1 KB (each column's sum is its own chain either way)
  const int pv_lo = F32 ? lane * 4 : lane * 8, pv_hi = F32 ? 256 + lane * 4 : lane * 8 + 4;
  float M[HG], Z[HG], O[HG][8];
#pragma unroll
  for (int h = 0; h < HG; ++h) {
    M[h] = -__builtin_inff();
    Z[h] = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) O[h][e] = 0.0f;
  }
  for (int tile = span * a.span_tiles; tile < tile_end; ++tile) {
    const int t0 = tile << 6, n = min(64, seq - t0);
    // stage rows t0 .. t0+n-1: 72 pieces of 16 bytes per row, 18 per thread
    {
      const uint4 *src = (const uint4 *)(cache + (size_t)t0 * KVA);
      constexpr int NP = (64 * 72 + W * 64 - 1) / (W * 64);  // pieces per thread: 18 with four waves
      uint4 v[NP];
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int idx = threadIdx.x + i * (W * 64);  // piece (row, j) = (idx / 72, idx % 72)
        v[i] = idx < n * 72 ? src[idx] : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const int idx = threadIdx.x + i * (W * 64), row = idx / 72, j = idx - row * 72;
        if ((64 * 72) % (W * 64) == 0 || idx < 64 * 72) {
          if (F32) {
            float cf[8];
            unpack8(cf, v[i]);
            float4 *dst = (float4 *)(tile_f + row * PITCH_F + j * 8);
            dst[0] = make_float4(cf[0], cf[1], cf[2], cf[3]);
            dst[1] = make_float4(cf[4], cf[5], cf[6], cf[7]);
          } else {
            *(uint4 *)(tile_lds + row * PITCH + j * 8) = v[i];
          }
        }
      }
    }
    __syncthreads();
    // 8 values of row r from column c_lo and (F32) c_hi on: a float4 each, so that 64 lanes read 1 KB in a row
    auto tile8 = [&](float (&cf)[8], int r, int c_lo, int c_hi) {
      if (F32) {
        const float4 lo = *(const float4 *)(tile_f + r * PITCH_F + c_lo), hi = *(const float4 *)(tile_f + r * PITCH_F + c_hi);
        cf[0] = lo.x; cf[1] = lo.y; cf[2] = lo.z; cf[3] = lo.w; cf[4] = hi.x; cf[5] = hi.y; cf[6] = hi.z; cf[7] = hi.w;
      } else {
        unpack8(cf, *(const uint4 *)(tile_lds + r * PITCH + c_lo));
      }
    };
    // scores: lane = position, one fma chain over the 576 columns per head
    float acc[HG];
#pragma unroll
    for (int h = 0; h < HG; ++h) acc[h] = 0.0f;
#pragma unroll 4
    for (int j = 0; j < KVA / 8; ++j) {
      float cf[8];
      tile8(cf, lane, j * 8, j * 8 + 4);
#pragma unroll
      for (int h = 0; h < HG; ++h) {
        const float *qh = q + h * KVA + j * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h] = __builtin_fmaf(cf[e], qh[e], acc[h]);
      }
    }
    float alpha[HG];
#pragma unroll
    for (int h = 0; h < HG; ++h) {
      float s = kx_bfround(kx_bfround(acc[h]) * a.rs * a.mscale * a.mscale);  // :429
      if (lane >= n) s = -__builtin_inff();
      const float mt = kxw::wave_max_f32(s);
      const float Mn = fmaxf(M[h], mt);
      alpha[h] = kx_expf(M[h] - Mn);
      const float p = lane < n ? kx_expf(s - Mn) : 0.0f;
      float z[1] = {p};
      kxw::reduce<1, 64>(z, lane);
      const float zt = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, z[0])));
      Z[h] = __builtin_fmaf(Z[h], alpha[h], zt);
      M[h] = Mn;
      p_lds[wave][h][lane] = kx_bfround(p);
    }
    // PV: lane = 8 latent columns (pv_lo .. +3 and pv_hi .. +3 as floats, pv_lo .. +7 as bf16), positions in order (p of
    // this wave was written by this wave)
#pragma unroll
    for (int h = 0; h < HG; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) O[h][e] = O[h][e] * alpha[h];
    // all 64 rows: rows past the sequence are staged as zeros and carry p = 0, which leaves O unchanged
#pragma unroll 8
    for (int t = 0; t < 64; ++t) {
      float cf[8];
      tile8(cf, t, pv_lo, pv_hi);
#pragma unroll
      for (int h = 0; h < HG; ++h) {
        const float p = p_lds[wave][h][t];
#pragma unroll
        for (int e = 0; e < 8; ++e) O[h][e] = __builtin_fmaf(p, cf[e], O[h][e]);
      }
    }
    __syncthreads();  // the next tile overwrites the staged rows
  }
#pragma unroll
  for (int h = 0; h < HG; ++h) {
    if (!h_valid) break;
    const size_t idx = ((size_t)b * a.spans + span) * a.heads + h0 + h;
    if (lane == 0) { a.pm[idx] = M[h]; a.pz[idx] = Z[h]; }
    *(float4 *)(a.po + idx * R + pv_lo) = make_float4(O[h][0], O[h][1], O[h][2], O[h][3]);
    *(float4 *)(a.po + idx * R + pv_hi) = make_float4(O[h][4], O[h][5], O[h][6], O[h][7]);
  }
}

// ---- the same partials on the matrix cores, for long contexts -----------------------------------
// q_abs and p = bf(exp(s - m)) are bf16-representable and the cache is bf16, so q.c and p.c are exact
// products summed in fp32: v_mfma_f32_32x32x16_bf16 computes what mla_partial_k computes with another
// summation order (held to the 1e-2 bar, not bit-exact; the token-identity runs use mla_partial_k).
// Workgroup = (sequence, span), 8 waves, 32-position tiles staged in LDS at their natural layout.  The two products
// run on different waves: waves 0-3 compute the scores of tile t, waves 4-7 the second product of tile t-1, and every
// SIMD holds one wave of each kind, so the matrix cores are fed from one wave while the other exponentiates, reads
// its operands or waits at a barrier:
//  * scores: wave (hb, kh) computes S^T[32 positions, heads 32 hb .. +31] over K steps 18 kh .. +17 of the 36 with
//    v_mfma_f32_32x32x16_bf16 (A = the 32 cache rows of the tile, one row per lane and 16-byte piece 2 ks + half;
//    B = the lane's head of q).  Every operand row is read by two waves.  Wave kh then takes heads 16 kh .. +15 of
//    the block: the sums of the other 16 heads go to the other wave through LDS, and the lanes that held them take
//    over half the positions of the wave's own heads, so all 32 positions of a head sit in four lanes of one wave:
//    maximum, exponentials, row sum and the running sum Z need no exchange between waves.  The wave writes
//    p = bf(exp(s - m)) at the K indices the second product reads them from, and exp(M_old - M_new);
//  * O^T[col, head] += C^T[col, pos] P^T[pos, head]: wave cq owns latent columns 128 cq .. +127 for all 64 heads
//    (two K steps per tile).  The A operand needs 8 positions of one column; ds_read_b64_tr_b16 delivers them from
//    the row-major tile: within 16 lanes, lane i points at four consecutive columns of row i / 4, and lane j
//    receives column j of the four rows.  The transposed reads of a tile are done once per column block and used
//    for both head blocks;
//  * two barriers per tile: behind the first, tile t has landed and p and the factors of tile t-1 are complete;
//    behind the second, the score sums are visible, and p and the operands of tile t-1 are in the registers of the
//    waves that use them: its ring buffer is free;
//  * the 32 cache rows of a tile are copied global -> LDS (no registers) by the waves of the second product, which
//    have the time, three tiles ahead into a ring of four buffers; rows sit at their natural pitch of 1152 B with
//    the 16-byte pieces xor-swizzled by the row, so the row-per-lane operand reads of the scores are free of bank
//    conflicts (counted: none), and a transposing read touches rows that differ in bit 3 of the position in its
//    two lane halves, which spreads it over all banks.
// An earlier form had all eight waves do both products (scores as 16 x 16 blocks, four waves reading every
// operand row, the maxima exchanged between waves): 0.54-0.55 ms against 0.52 ms at 16 sequences of 131072
// positions, 56 against 49 us at 32 sequences of 4096.
constexpr int MM_T = 32;                      // positions per tile
constexpr int MM_NAT = MM_T * MLA_KVA * 2;    // bytes of one staged tile
constexpr int MM_RING = 4;
constexpr int MM_P_PITCH = 80;                // bytes per head of the staged probabilities: 32 positions + pad
constexpr int MM_LDS = MM_RING * MM_NAT;     // dynamic part: the tile ring
typedef float kx_f32x16v __attribute__((ext_vector_type(16)));
typedef __bf16 kx_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 kx_bf16x2v __attribute__((ext_vector_type(2)));
typedef float kx_f32x2v __attribute__((ext_vector_type(2)));
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 kx_bf16x4t;
// two f32 -> packed bf16 pair, round to nearest even (v_cvt_pk_bf16_f32; the same values as kx_bf16_rne for finite inputs)
__device__ __forceinline__ uint32_t mm_pack_bf16(float lo, float hi) {
  kx_f32x2v v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, kx_bf16x2v));
}
// ds_read_b64_tr_b16 at LDS byte address `addr`
__device__ __forceinline__ uint2 mm_read_tr(uint32_t addr) {
  kx_bf16x4t v = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) kx_bf16x4t *)(uintptr_t)addr);
  return __builtin_bit_cast(uint2, v);
}
// the copies into the tile ring and the fence-free barrier: kx_lds_copy.h (this kernel waits for a tile itself,
// where it needs it: wait_tile below)
__device__ __forceinline__ void mm_copy16_to_lds(const void *src, uint32_t lds_base) { kx_copy16_to_lds(src, lds_base); }
__device__ __forceinline__ void mm_barrier() { kx_lds_barrier(); }

__global__ void __launch_bounds__(512, 1) mla_partial_mfma_k(MlaArgs a) {
  extern __shared__ __attribute__((aligned(128))) uint8_t mm_lds[];
  uint8_t *nat = mm_lds;                       // [4][32 rows][72 pieces of 16 B]
  __shared__ __attribute__((aligned(16))) uint8_t p_lds[64 * MM_P_PITCH];    // [64 heads]: bf16 p by K index
  __shared__ __attribute__((aligned(16))) float sp_lds[2 * 2 * 4 * 32 * 4];  // [hb][kh][q][16 half + head % 16]: score sums of wave (hb, kh) for the other wave's heads
  __shared__ float al_lds[64];                 // [64] exp(M_old - M_new)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int span = blockIdx.x, b = blockIdx.z;
  const int l32 = lane & 31, half = lane >> 5;
  const bool scorer = wave < 4;
  const int hb = wave & 1, kh = (wave >> 1) & 1;  // score waves
  const int cq = wave & 3;                        // waves of the second product
  const int seq = a.seqs ? a.seq - (int)(gridDim.z / a.seqs) + 1 + b / a.seqs : a.seq;
  const uint16_t *cache = a.cache + (size_t)(a.seqs ? b % a.seqs : b) * a.seq_stride;
  const int pos0 = span * a.span_tiles * 64, pos_end = min(seq, (span + 1) * a.span_tiles * 64);
  if (pos0 >= seq) {  // a span past this position's rows (prefill steps only): partials the merge weighs with 0
    const size_t base = ((size_t)b * a.spans + span) * a.heads;
    if (threadIdx.x < (unsigned)a.heads) { a.pm[base + threadIdx.x] = -__builtin_inff(); a.pz[base + threadIdx.x] = 0.0f; }
    for (int i = threadIdx.x; i < a.heads * 512; i += 512) a.po[base * 512 + i] = 0.0f;
    return;
  }
  const int n_tiles = (pos_end - pos0 + MM_T - 1) / MM_T;
  const float scale = a.rs * a.mscale * a.mscale;
  constexpr float LOG2E = 1.44269504088896341f;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)nat;

  // global -> LDS copy of a tile by the four waves of the second product, which have the time: 2304 pieces = 36
  // instructions, nine per wave; slot (row p, j') holds piece j' ^ ((p >> 1) & 7) (low three bits) of the row; rows past
  // the sequence repeat its last row.  The lane's places inside a tile do not change from tile to tile: the nine
  // source offsets are kept, and only a tile that reaches past the sequence goes through the row clamp.
  const int cw = wave & 3;
  int c_off[9];   // elements from the tile's first row
  int c_row[9];
#pragma unroll
  for (int u = 0; u < 9; ++u) {
    const int slot = (cw + 4 * u) * 64 + lane;
    const int p = slot / 72, js = slot - p * 72;
    const int j = (js & ~7) | ((js ^ (p >> 1)) & 7);
    c_row[u] = p;
    c_off[u] = p * MLA_KVA + j * 8;
  }
  auto copy_tile = [&](int t) {
    const int row0 = pos0 + t * MM_T;
    const uint16_t *src = cache + (size_t)row0 * MLA_KVA;
    const uint32_t dst = lds0 + (t % MM_RING) * MM_NAT + cw * 1024;
    if (row0 + MM_T <= seq) {
#pragma unroll
      for (int u = 0; u < 9; ++u) mm_copy16_to_lds(src + c_off[u], dst + u * 4096);
    } else {
#pragma unroll
      for (int u = 0; u < 9; ++u) {
        const int back = max(row0 + c_row[u] - (seq - 1), 0);  // rows past the last one
        mm_copy16_to_lds(src + c_off[u] - back * MLA_KVA, dst + u * 4096);
      }
    }
  };
  // Tile t + 3 is requested behind the second barrier of iteration t, into the ring buffer of tile t - 1 (whose
  // operands are in registers by then).  At the top of iteration t the copies of tiles t + 1 and t + 2, nine each,
  // are the wave's newest: tile t has landed when only they are outstanding.
  auto wait_tile = [&](int t) {
    if (t + 2 < n_tiles) asm volatile("s_waitcnt vmcnt(18)" ::: "memory");
    else if (t + 1 < n_tiles) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };

  if (!scorer) {
    copy_tile(0);
    if (n_tiles > 1) copy_tile(1);
    if (n_tiles > 2) copy_tile(2);
  }
  // One loop per kind of wave, with the same barriers in the same order: the registers of one kind (q, 72; the
  // output blocks, 128) are then not live in the other's loop.
  if (scorer) {
    // q of head 32 hb + l32 as B operands; K step 18 kh + i covers columns 16 (18 kh + i) + 8 half .. +7
    kx_bf16x8 qf[18];
    {
      const float *q = a.qabs + ((size_t)b * a.heads + hb * 32 + l32) * MLA_KVA + kh * 288 + half * 8;
#pragma unroll
      for (int i = 0; i < 18; ++i) {
        const float4 lo = *(const float4 *)(q + i * 16), hi = *(const float4 *)(q + i * 16 + 4);
        const uint4 u = make_uint4((kx_f32_bits(lo.x) >> 16) | (kx_f32_bits(lo.y) & 0xffff0000u),
                                   (kx_f32_bits(lo.z) >> 16) | (kx_f32_bits(lo.w) & 0xffff0000u),
                                   (kx_f32_bits(hi.x) >> 16) | (kx_f32_bits(hi.y) & 0xffff0000u),
                                   (kx_f32_bits(hi.z) >> 16) | (kx_f32_bits(hi.w) & 0xffff0000u));
        qf[i] = __builtin_bit_cast(kx_bf16x8, u);
      }
    }
    // A operands: row l32, piece 2 ks + half = 8 (ks / 4) + (2 (ks % 4) + half) with ks = 18 kh + i; s_off[u] is the
    // swizzled place of piece 2 u + half inside its group of eight
    int s_off[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) s_off[u] = l32 * (MLA_KVA * 2) + (((2 * u + half) ^ (l32 >> 1)) & 7) * 16;
    // After the products, wave kh keeps heads 16 kh .. +15 of the block.  Its lanes with the other wave's heads
    // (row = lane / 16 odd for kh = 0, even for kh = 1) put their sums into LDS for that wave and then take over
    // positions 16 .. 31 of the head 16 lanes away (v_permlane16_swap), so that every lane has eight positions of a
    // head of the wave: lane = (head 16 kh + lane % 16, half, qsel), positions 8 q + 4 half + c with q = 2 qsel + j / 4,
    // c = j % 4 for value j.
    const int h16 = lane & 15;
    const int qsel = ((l32 >> 4) != kh) ? 1 : 0;
    const int headx = hb * 32 + kh * 16 + h16;
    float M = -__builtin_inff(), Z = 0.0f;  // of headx; the four lanes of a head keep identical copies
    kx_f32x16v sacc;
    float v[8];
    auto scores = [&](auto k_first, const uint8_t *st) {
      constexpr int K0 = decltype(k_first)::value;
      constexpr int AH = 3;
      kx_bf16x8 av[AH + 1];
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[i] = 0.0f;
#pragma unroll
      for (int i = 0; i < AH; ++i) av[i] = *(const kx_bf16x8 *)(st + s_off[(K0 + i) & 3] + ((K0 + i) >> 2) * 128);
#pragma unroll
      for (int i = 0; i < 18; ++i) {
        if (i + AH < 18)
          av[(i + AH) % (AH + 1)] = *(const kx_bf16x8 *)(st + s_off[(K0 + i + AH) & 3] + ((K0 + i + AH) >> 2) * 128);
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[i % (AH + 1)], qf[i], sacc, 0, 0, 0);
      }
      // accumulator 4 q + c of lane (head l32, half) is position 8 q + 4 half + c
      if (qsel) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *(float4 *)(sp_lds + ((((hb * 2 + kh) * 4 + q) * 32) + 16 * half + h16) * 4) =
              make_float4(sacc[4 * q], sacc[4 * q + 1], sacc[4 * q + 2], sacc[4 * q + 3]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float x = sacc[j], y = sacc[8 + j];
        if (K0 == 0) {  // rows 1, 3 of x <- rows 0, 2 of y
          kxw::swap_rows16(x, y);
          v[j] = x;
        } else {        // rows 0, 2 of x <- rows 1, 3 of y
          kxw::swap_rows16(y, x);
          v[j] = x;
        }
      }
    };
    auto softmax_tile = [&](int t) {
      float sv[8];
      float mloc = -__builtin_inff();
#pragma unroll
      for (int qq = 0; qq < 2; ++qq) {
        const int q = 2 * qsel + qq;
        const float4 o = *(const float4 *)(sp_lds + ((((hb * 2 + (kh ^ 1)) * 4 + q) * 32) + 16 * half + h16) * 4);
        const float sum[4] = {v[4 * qq] + o.x, v[4 * qq + 1] + o.y, v[4 * qq + 2] + o.z, v[4 * qq + 3] + o.w};
#pragma unroll
        for (int c = 0; c < 4; c += 2) {
          const int pos = pos0 + t * MM_T + 8 * q + 4 * half + c;
          const uint32_t r0 = mm_pack_bf16(sum[c], sum[c + 1]);                                                     // bf(q.k)
          const uint32_t r1 = mm_pack_bf16(kx_bits_f32(r0 << 16) * scale, kx_bits_f32(r0 & 0xffff0000u) * scale);  // bf(. * scale)
          float s0 = kx_bits_f32(r1 << 16), s1 = kx_bits_f32(r1 & 0xffff0000u);
          if (pos >= pos_end) s0 = -__builtin_inff();
          if (pos + 1 >= pos_end) s1 = -__builtin_inff();
          sv[4 * qq + c] = s0;
          sv[4 * qq + c + 1] = s1;
          mloc = fmaxf(mloc, fmaxf(s0, s1));
        }
      }
      {  // maximum over the four lanes of the head: lanes l ^ 16 and l ^ 32
        float o = mloc;
        kxw::swap_rows16(mloc, o);
        mloc = fmaxf(mloc, o);
        o = mloc;
        kxw::swap_halves32(mloc, o);
        mloc = fmaxf(mloc, o);
      }
      const float Mn = fmaxf(M, mloc);
      const float alpha = __builtin_amdgcn_exp2f((M - Mn) * LOG2E);
      float e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = __builtin_amdgcn_exp2f((sv[i] - Mn) * LOG2E);
      float ps = ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
      {
        float o = ps;
        kxw::swap_rows16(ps, o);
        ps += o;
        o = ps;
        kxw::swap_halves32(ps, o);
        ps += o;
      }
      // the lane's positions are those of MFMA step qsel; inside the step position 8 (q % 2) + 4 half + c sits at K index
      // 8 half + 4 (c / 2) + 2 (q % 2) + (c % 2): one 16-byte piece per lane
      *(uint4 *)(p_lds + headx * MM_P_PITCH + qsel * 32 + half * 16) =
          make_uint4(mm_pack_bf16(e[0], e[1]), mm_pack_bf16(e[4], e[5]), mm_pack_bf16(e[2], e[3]), mm_pack_bf16(e[6], e[7]));
      if (half == 0 && qsel == 0) al_lds[headx] = alpha;
      Z = __builtin_fmaf(Z, alpha, ps);
      M = Mn;
    };
    for (int t = 0; t <= n_tiles; ++t) {
      mm_barrier();  // tile t has landed (the copying waves have waited for it); p and the factors of tile t-1 are complete
      if (t < n_tiles) {
        const uint8_t *st = nat + (t % MM_RING) * MM_NAT;
        if (kh == 0) scores(std::integral_constant<int, 0>{}, st);
        else scores(std::integral_constant<int, 18>{}, st);
      }
      mm_barrier();  // the score sums are visible; p of tile t-1 is in the registers of the other waves
      if (t < n_tiles) softmax_tile(t);
    }
    if (half == 0 && qsel == 0) {
      const size_t idx = ((size_t)b * a.spans + span) * a.heads + headx;
      a.pm[idx] = M;
      a.pz[idx] = Z;
    }
  } else {
    // transposing reads of the second product: as in mla_partial_mfma_k
    int t_off[2][2];
    {
      const int i = lane & 15, grp = (lane >> 4) & 1;
#pragma unroll
      for (int sidx = 0; sidx < 2; ++sidx)
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          const int p = 16 * sidx + 4 * half + 2 * w + ((i >> 2) & 1) + 8 * (i >> 3);
          const int low3 = 2 * grp + ((i >> 1) & 1);
          t_off[sidx][w] = p * (MLA_KVA * 2) + (2 * cq) * 128 + ((low3 ^ (p >> 1)) & 7) * 16 + (i & 1) * 8;
        }
    }
    kx_f32x16v O[2][4];  // [head block][cbk]: heads x columns 128 cq + 32 cbk .. +31
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
      for (int cbk = 0; cbk < 4; ++cbk)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[h2][cbk][i] = 0.0f;
    kx_bf16x8 pf[2][2], pa[8];
    // what the second product of a tile needs from LDS: p of both head blocks, the factors, the transposed operands
    auto pv_begin = [&](uint32_t sp) {
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        pf[h2][0] = *(const kx_bf16x8 *)(p_lds + (h2 * 32 + l32) * MM_P_PITCH + half * 16);
        pf[h2][1] = *(const kx_bf16x8 *)(p_lds + (h2 * 32 + l32) * MM_P_PITCH + 32 + half * 16);
        const float alpha2 = al_lds[h2 * 32 + l32];
        if (__builtin_amdgcn_ballot_w64(alpha2 != 1.0f) != 0) {  // the running maximum of some head of the block moved
          asm volatile("" ::: "memory");                          // keep this a branch: it is rarely taken after the first tiles
#pragma unroll
          for (int cbk = 0; cbk < 4; ++cbk) O[h2][cbk] *= alpha2;
        }
      }
#pragma unroll
      for (int sidx = 0; sidx < 2; ++sidx) {
        const uint32_t a0 = sp + t_off[sidx][0], a1 = sp + t_off[sidx][1];
        const uint32_t b0 = sp + (t_off[sidx][0] ^ 64), b1 = sp + (t_off[sidx][1] ^ 64);
        const uint2 l0 = mm_read_tr(a0), h0 = mm_read_tr(a1), l1 = mm_read_tr(b0), h1 = mm_read_tr(b1);
        const uint2 l2 = mm_read_tr(a0 + 128), h2 = mm_read_tr(a1 + 128), l3 = mm_read_tr(b0 + 128), h3 = mm_read_tr(b1 + 128);
        pa[0 + sidx] = __builtin_bit_cast(kx_bf16x8, make_uint4(l0.x, l0.y, h0.x, h0.y));
        pa[2 + sidx] = __builtin_bit_cast(kx_bf16x8, make_uint4(l1.x, l1.y, h1.x, h1.y));
        pa[4 + sidx] = __builtin_bit_cast(kx_bf16x8, make_uint4(l2.x, l2.y, h2.x, h2.y));
        pa[6 + sidx] = __builtin_bit_cast(kx_bf16x8, make_uint4(l3.x, l3.y, h3.x, h3.y));
      }
    };
    auto pv_mfma = [&](int m0, int m1) {
#pragma unroll
      for (int m = 0; m < 8; ++m)
        if (m >= m0 && m < m1) {
          O[0][m >> 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pa[m], pf[0][m & 1], O[0][m >> 1], 0, 0, 0);
          O[1][m >> 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pa[m], pf[1][m & 1], O[1][m >> 1], 0, 0, 0);
        }
    };
    for (int t = 0; t <= n_tiles; ++t) {
      if (t < n_tiles) wait_tile(t);
      mm_barrier();
      if (t > 0) pv_begin(lds0 + ((t - 1) % MM_RING) * MM_NAT);
      mm_barrier();
      if (t + 3 < n_tiles) copy_tile(t + 3);
      if (t > 0) pv_mfma(0, 8);
    }
    // O: lane = (head, column 128 cq + 32 cbk + 8 q + 4 half + c) for accumulator register 4 q + c
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      const size_t idx2 = ((size_t)b * a.spans + span) * a.heads + h2 * 32 + l32;
#pragma unroll
      for (int cbk = 0; cbk < 4; ++cbk)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *(float4 *)(a.po + idx2 * MLA_R + cq * 128 + cbk * 32 + q * 8 + half * 4) =
              make_float4(O[h2][cbk][4 * q], O[h2][cbk][4 * q + 1], O[h2][cbk][4 * q + 2], O[h2][cbk][4 * q + 3]);
    }
  }
}

// merge of the spans; grid (heads, B), one wave, lane = 8 latent columns
__global__ void __launch_bounds__(64) mla_combine_k(const float *__restrict__ pm, const float *__restrict__ pz,
                                                    const float *__restrict__ po, uint16_t *__restrict__ o_lat, int heads,
                                                    int spans) {
  // M = max M_j; w_j = exp(M_j - M); Z = fma(Z_j, w_j, Z); O = fma(O_j, w_j, O) in span order.  Spans are taken in
  // groups of 64: lane j holds (M_j, Z_j, w_j) of the group's span j; the O_j rows are fetched sixteen at a time.
  constexpr int R = 512;
  const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  const size_t idx0 = (size_t)b * spans * heads + h;
  float M = -__builtin_inff();
  for (int g0 = 0; g0 < spans; g0 += 64) {
    const float mj = g0 + lane < spans ? pm[idx0 + (size_t)(g0 + lane) * heads] : -__builtin_inff();
    M = fmaxf(M, kxw::wave_max_f32(mj));
  }
  float Z = 0.0f, O[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int g0 = 0; g0 < spans; g0 += 64) {
    const int gn = min(64, spans - g0);
    const size_t my = idx0 + (size_t)(g0 + min(lane, gn - 1)) * heads;
    const float mj = pm[my], zj = pz[my];
    const float wj = kx_expf(mj - M);
    for (int j = 0; j < gn; ++j)
      Z = __builtin_fmaf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, zj), j)),
                         __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), j)), Z);
    for (int j0 = 0; j0 < gn; j0 += 16) {
      float4 o0[16], o1[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const float4 *o = (const float4 *)(po + (idx0 + (size_t)(g0 + min(j0 + u, gn - 1)) * heads) * R + lane * 8);
        o0[u] = o[0];
        o1[u] = o[1];
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        if (j0 + u < gn) {
          const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), j0 + u));
          O[0] = __builtin_fmaf(o0[u].x, w, O[0]); O[1] = __builtin_fmaf(o0[u].y, w, O[1]);
          O[2] = __builtin_fmaf(o0[u].z, w, O[2]); O[3] = __builtin_fmaf(o0[u].w, w, O[3]);
          O[4] = __builtin_fmaf(o1[u].x, w, O[4]); O[5] = __builtin_fmaf(o1[u].y, w, O[5]);
          O[6] = __builtin_fmaf(o1[u].z, w, O[6]); O[7] = __builtin_fmaf(o1[u].w, w, O[7]);
        }
      }
    }
  }
  uint32_t r[4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
    r[e] = (uint32_t)kx_bf16_rne(O[2 * e] / Z) | ((uint32_t)kx_bf16_rne(O[2 * e + 1] / Z) << 16);
  *(uint4 *)(o_lat + ((size_t)b * heads + h) * R + lane * 8) = make_uint4(r[0], r[1], r[2], r[3]);
}

// the same merge for few (sequence, head) pairs: grid (heads, B, 8), one wave per 64 latent columns, lane = one column
__global__ void __launch_bounds__(64) mla_combine_cols_k(const float *__restrict__ pm, const float *__restrict__ pz,
                                                    const float *__restrict__ po, uint16_t *__restrict__ o_lat, int heads,
                                                    int spans) {
  // M = max M_j; w_j = exp(M_j - M); Z = fma(Z_j, w_j, Z); O = fma(O_j, w_j, O) in span order.  Spans are taken in
  // groups of 64: lane j holds (M_j, Z_j, w_j) of the group's span j, and the group's 64 values of the lane's
  // column are requested together.
  constexpr int R = 512;
  const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  const int col = blockIdx.z * 64 + lane;
  const size_t idx0 = (size_t)b * spans * heads + h;
  float M = -__builtin_inff();
  for (int g0 = 0; g0 < spans; g0 += 64) {
    const float mj = g0 + lane < spans ? pm[idx0 + (size_t)(g0 + lane) * heads] : -__builtin_inff();
    M = fmaxf(M, kxw::wave_max_f32(mj));
  }
  float Z = 0.0f, O = 0.0f;
  for (int g0 = 0; g0 < spans; g0 += 64) {
    const int gn = min(64, spans - g0);
    const size_t my = idx0 + (size_t)(g0 + min(lane, gn - 1)) * heads;
    const float mj = pm[my], zj = pz[my];
    const float wj = kx_expf(mj - M);
    for (int j = 0; j < gn; ++j)
      Z = __builtin_fmaf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, zj), j)),
                         __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), j)), Z);
    float o[64];
#pragma unroll
    for (int u = 0; u < 64; ++u) o[u] = po[(idx0 + (size_t)(g0 + min(u, gn - 1)) * heads) * R + col];
#pragma unroll
    for (int u = 0; u < 64; ++u)
      if (u < gn) O = __builtin_fmaf(o[u], __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), u)), O);
  }
  o_lat[((size_t)b * heads + h) * R + col] = kx_bf16_rne(O / Z);
}

}  // namespace

int kx_q_absorb_launch(const uint16_t *q, const uint16_t *kvb, const uint16_t *rope_row, float *qabs, int tokens,
                       int heads, int nope, int rope, int v_head, int kv_rank, const uint16_t *kva, int kva_stride,
                       const uint16_t *w_kv_ln, uint16_t *cache, size_t seq_stride, int pos, float eps, hipStream_t st, int seqs) {
  KX_REQUIRE(kv_rank % 8 == 0 && kv_rank <= 1024 && rope % 2 == 0 && rope / 2 <= 128, "kx_q_absorb: kv_rank=%d (multiple of 8, at most 1024), rope=%d (even, at most 256)", kv_rank, rope);
  QAbsArgs a = {};
  a.q = q; a.kvb = kvb; a.rope_row = rope_row; a.qabs = qabs; a.kva = kva; a.w_kv_ln = w_kv_ln; a.cache = cache;
  a.seq_stride = seq_stride; a.heads = heads; a.nope = nope; a.rope = rope; a.v_head = v_head; a.kv_rank = kv_rank;
  a.kva_stride = kva_stride; a.pos = pos; a.eps = eps; a.seqs = seqs;
  KX_REQUIRE(seqs == 0 || (seqs > 0 && tokens % seqs == 0), "kx_q_absorb: %d tokens do not split into %d sequences", tokens, seqs);
  const dim3 g1(heads * ((kv_rank + 127) / 128) + (cache ? 1 : 0), tokens);
  if (tokens >= 64) hipLaunchKernelGGL(q_absorb_k<8>, dim3(g1.x, (tokens + 7) / 8), dim3(128), 0, st, a, tokens);
  else if (tokens >= 8) hipLaunchKernelGGL(q_absorb_k<4>, dim3(g1.x, (tokens + 3) / 4), dim3(128), 0, st, a, tokens);
  else hipLaunchKernelGGL(q_absorb_k<1>, g1, dim3(128), 0, st, a, tokens);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

size_t kx_mla_partial_floats(int batch, int heads, int kv_rank, int max_seq) {
  const int tiles = (max_seq + 63) / 64, st = kx_mla_span_tiles(max_seq);
  int spans = (tiles + st - 1) / st;
  if (spans < 64) spans = tiles < 64 ? tiles : 64;  // shorter sequences use up to 64 spans
  size_t rows = (size_t)batch * spans;              // (sequence, span) pairs of the fixed partition
  for (int b = 1; b <= batch; ++b) {                // and of the matrix-core kernel's, for every batch up to this one
    const int cap = mfma_span_cap(b);
    const size_t r = (size_t)b * (tiles < cap ? tiles : cap);
    if (r > rows) rows = r;
  }
  return rows * heads * (kv_rank + 2);
}

int kx_mla_partials_launch(const kx_config *c, const uint16_t *cache, size_t seq_stride, const float *qabs, float *partial,
                           int batch, int seq, KxMlaPartials *out, hipStream_t st, int seqs, int kernel) {
  KX_REQUIRE(kernel >= KX_MLA_AUTO && kernel <= KX_MLA_MATRIX_CORES, "kx_mla: kernel=%d outside [0, 2]", kernel);
  KX_REQUIRE(c->kv_rank == 512 && c->qk_rope == 64, "kx_mla: the attention kernel is built for kv_rank 512, qk_rope 64 (got %d, %d)",
             c->kv_rank, c->qk_rope);
  KX_REQUIRE(c->heads % 4 == 0, "kx_mla: heads=%d must be a multiple of 4", c->heads);
  KX_REQUIRE(batch > 0 && seq > 0, "kx_mla: batch=%d seq=%d must be positive", batch, seq);
  KX_REQUIRE(seqs == 0 || (seqs > 0 && batch % seqs == 0 && seq >= batch / seqs), "kx_mla: %d positions x sequences do not split into %d sequences of at least %d positions", batch, seqs, seq);
  // automatic choice, where the matrix-core kernel is built for the shape (64 heads): from 2048 positions on, and from
  // 128 positions on for 5 sequences and more (batches the stack runs on the matrix cores anyway; the VALU kernel
  // takes 190-360 us per layer at 32 sequences of 1100 positions)
  const bool use_mfma = kernel == KX_MLA_MATRIX_CORES || (kernel == KX_MLA_AUTO && c->heads == 64 && (seq >= 2048 || (batch >= 5 && seq >= 128)));
  MlaArgs a;
  a.cache = cache; a.qabs = qabs; a.heads = c->heads; a.seq = seq; a.seq_stride = seq_stride; a.seqs = seqs;
  a.span_tiles = use_mfma ? mfma_span_tiles(seq, batch) : kx_mla_span_tiles(seq);
  const int tiles = (seq + 63) / 64;
  a.spans = (tiles + a.span_tiles - 1) / a.span_tiles;
  const size_t n = (size_t)batch * a.spans * c->heads;
  a.pm = partial; a.pz = partial + n; a.po = partial + 2 * n;
  float rs, ms;
  kx_softmax_scale(c, &rs, &ms);
  a.rs = rs; a.mscale = ms;
  // heads per wave: enough waves to fill the chip, as few as possible otherwise
  const long waves1 = (long)batch * a.spans * c->heads;  // waves at one head per wave
  int hg = 1;
  while (hg < 8 && c->heads % (4 * hg * 2) == 0 && waves1 / (hg * 2) >= 4096) hg *= 2;
  // One head per wave and more workgroups of four waves than CUs, but not many more (a context of 1100 positions and
  // one sequence: 18 spans x 16 = 288): the CUs that get two take half as long again as the rest, and that is the
  // launch.  Six to eight waves per workgroup -- fewer, wider workgroups that share a tile among more heads -- where
  // that brings the launch to one workgroup per CU.  (Measured on the decode steps of the 24-layer stack at 1030-1290
  // positions, tok/s: four waves 247.7, five 248.7 where they fit, six 251.2, seven 248.8, eight 248.9.)
  int wv = 4;
  if (hg == 1 && !use_mfma && (long)batch * a.spans * (c->heads / 4) > mla_compute_units()) {
    for (int w = 6; w <= 8 && wv == 4; ++w)
      if ((long)batch * a.spans * kx_cdiv(c->heads, w) <= mla_compute_units()) wv = w;
  }
  dim3 g(a.spans, kx_cdiv(c->heads, wv * hg), batch), b(wv * 64);
  // one workgroup per CU at most: the tile as floats (see the kernel)
  const bool f32 = hg == 1 && !use_mfma && (long)g.x * g.y * g.z <= mla_compute_units();
  const size_t lds = f32 ? (size_t)64 * MLA_PITCH_F * 4 + (size_t)wv * 64 * sizeof(float)
                         : (size_t)64 * MLA_PITCH * 2 + (size_t)wv * hg * 64 * sizeof(float);
  static std::atomic<bool> attr_set{false};  // setting it twice from two threads is harmless
  if (!attr_set) {  // more than 64 KB of dynamic LDS has to be allowed per kernel
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<1, 6>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<1, 7>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<1, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<2>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<4>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<1, 4, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<1, 6, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<1, 7, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024));
    KX_HIP(hipFuncSetAttribute((const void *)mla_partial_k<1, 8, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024));
    attr_set = true;
  }
  if (use_mfma) {
    KX_REQUIRE(c->heads == 64, "kx_mla: the matrix-core kernel is built for 64 heads (got %d)", c->heads);
    static std::atomic<bool> mfma_attr{false};
    if (!mfma_attr) {
      KX_HIP(hipFuncSetAttribute((const void *)mla_partial_mfma_k, hipFuncAttributeMaxDynamicSharedMemorySize, MM_LDS));
      mfma_attr = true;
    }
    hipLaunchKernelGGL(mla_partial_mfma_k, dim3(a.spans, 1, batch), dim3(512), MM_LDS, st, a);
    KX_LAUNCH_CHECK();
    out->pm = a.pm; out->pz = a.pz; out->po = a.po; out->spans = a.spans;
    return KX_OK;
  }
  if (f32 && wv == 4) hipLaunchKernelGGL((mla_partial_k<1, 4, true>), g, b, lds, st, a);
  else if (f32 && wv == 6) hipLaunchKernelGGL((mla_partial_k<1, 6, true>), g, b, lds, st, a);
  else if (f32 && wv == 7) hipLaunchKernelGGL((mla_partial_k<1, 7, true>), g, b, lds, st, a);
  else if (f32 && wv == 8) hipLaunchKernelGGL((mla_partial_k<1, 8, true>), g, b, lds, st, a);
  else if (hg == 1 && wv == 6) hipLaunchKernelGGL((mla_partial_k<1, 6>), g, b, lds, st, a);
  else if (hg == 1 && wv == 7) hipLaunchKernelGGL((mla_partial_k<1, 7>), g, b, lds, st, a);
  else if (hg == 1 && wv == 8) hipLaunchKernelGGL((mla_partial_k<1, 8>), g, b, lds, st, a);
  else if (hg == 1) hipLaunchKernelGGL(mla_partial_k<1>, g, b, lds, st, a);
  else if (hg == 2) hipLaunchKernelGGL(mla_partial_k<2>, g, b, lds, st, a);
  else if (hg == 4) hipLaunchKernelGGL(mla_partial_k<4>, g, b, lds, st, a);
  else hipLaunchKernelGGL(mla_partial_k<8>, g, b, lds, st, a);
  KX_LAUNCH_CHECK();
  out->pm = a.pm; out->pz = a.pz; out->po = a.po; out->spans = a.spans;
  return KX_OK;
}

int kx_mla_combine_launch(const KxMlaPartials &p, uint16_t *o_lat, int batch, int heads, hipStream_t st) {
  if ((long)heads * batch < 512)  // few waves: a wave per 64 columns, all of a group's rows in flight
    hipLaunchKernelGGL(mla_combine_cols_k, dim3(heads, batch, 8), dim3(64), 0, st, p.pm, p.pz, p.po, o_lat, heads, p.spans);
  else
    hipLaunchKernelGGL(mla_combine_k, dim3(heads, batch), dim3(64), 0, st, p.pm, p.pz, p.po, o_lat, heads, p.spans);
  KX_LAUNCH_CHECK();
  return KX_OK;
}

int kx_mla_attend_launch(const kx_config *c, const uint16_t *cache, size_t seq_stride, const float *qabs, float *partial,
                         uint16_t *o_lat, int batch, int seq, hipStream_t st, int seqs, int kernel) {
  KxMlaPartials p;
  int rc = kx_mla_partials_launch(c, cache, seq_stride, qabs, partial, batch, seq, &p, st, seqs, kernel);
  if (rc) return rc;
  return kx_mla_combine_launch(p, o_lat, batch, c->heads, st);
}

// ---- C ABI: BASELINE config 3 as an operator -------------------------------------------
extern "C" int kx_mla_workspace_bytes(const kx_config *cfg, int32_t batch, int32_t max_seq, size_t *bytes) {
  KX_REQUIRE(cfg && bytes, "kx_mla_workspace_bytes: null argument");
  KX_REQUIRE(batch > 0 && max_seq > 0, "kx_mla_workspace_bytes: batch=%d max_seq=%d must be positive", batch, max_seq);
  *bytes = kx_mla_partial_floats(batch, cfg->heads, cfg->kv_rank, max_seq) * sizeof(float);
  return KX_OK;
}

extern "C" int kx_mla_decode(const kx_config *cfg, const void *d_cache, size_t seq_stride, const void *d_qabs,
                             void *d_workspace, void *d_o_lat, int32_t batch, int32_t seq, int32_t kernel, void *stream) {
  KX_REQUIRE(cfg && d_cache && d_qabs && d_workspace && d_o_lat, "kx_mla_decode: null argument");
  KX_REQUIRE(seq_stride >= (size_t)seq * (cfg->kv_rank + cfg->qk_rope), "kx_mla_decode: seq_stride shorter than the sequence");
  return kx_mla_attend_launch(cfg, (const uint16_t *)d_cache, seq_stride, (const float *)d_qabs, (float *)d_workspace,
                              (uint16_t *)d_o_lat, batch, seq, kx_stream(stream), 0, kernel);
}

extern "C" int kx_q_absorb(const kx_config *cfg, const void *d_q, const void *d_kvb, const void *d_rope_row, void *d_qabs,
                           int32_t tokens, void *stream) {
  KX_REQUIRE(cfg && d_q && d_kvb && d_rope_row && d_qabs, "kx_q_absorb: null argument");
  return kx_q_absorb_launch((const uint16_t *)d_q, (const uint16_t *)d_kvb, (const uint16_t *)d_rope_row, (float *)d_qabs,
                            tokens, cfg->heads, cfg->qk_nope, cfg->qk_rope, cfg->v_head, cfg->kv_rank, nullptr, 0, nullptr,
                            nullptr, 0, 0, 0.0f, kx_stream(stream));
}
