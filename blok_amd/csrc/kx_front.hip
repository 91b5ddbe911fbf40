// kx_front.hip -- the two halves of the attention block around the attention itself, for one token, as one resident
// launch each (the back: attn_back_k below).  The front:
//   q_a GEMV with the input RMSNorm      (src/kimi_exec.cu:812-813)
//   q_b GEMV with the q_a RMSNorm        (:814-815)
//   kv_a GEMV, its RMSNorm, RoPE of the shared key, the cache row   (:816-817, :820-824)
//   q_abs = (bf(W_UK^T q_nope) | rope(q_rope)) per head             (:818 as W_UK, rope_k :346-357)
// The reference runs these as seven launches with a tile read from NVMe in front of each; the separate-launch
// form of this library runs them as two (gemv_bf16_k for q_a|kv_a, gemv_absorb_k).  q_b needs all of q_a and the
// absorb needs a whole head of q, so the steps are a chain, and as launches each of them pays its start and its
// drain while the memory system idles.  Here one workgroup per CU stays resident, and its 48 rows of q_b (144 KB)
// are copied global -> LDS while q_a travels between the workgroups, so that the q_b step reads them at LDS speed.
//
//   every workgroup: 6 rows of q_a and 2 or 3 of kv_a, all loads out at once (waves 0..6) -> hand the 8 or 9 values
//                    over; waves 4..7 start the copy of the workgroup's 48 rows of q_b into LDS -> take all of q_a ->
//                    q rows [48 b, 48 b + 48) from LDS -> hand them over -> (workgroup 0: take kv_a, norm, RoPE,
//                    cache row) -> take its head's q -> a quarter of the head's q_abs
//
// Sums are the ones of the separate-launch kernels (kx_gemv_body.h, kx_attn_parts.h): results are equal to the
// bit, which the fused / separate test of the stack checks.
//
// Hand-over between workgroups: no barrier and no counter.  A value travels as one 32-bit word that carries the
// launch's tag above its bf16 bits; the reader polls the words it needs until they carry the tag.  A word is one
// relaxed atomic object, so nothing has to be ordered, acknowledged or reset.  All workgroups must be resident at
// once (a reader waits for writers): the launcher refuses a device with fewer CUs than workgroups, and the LDS a
// workgroup takes keeps a second one off its CU.  The wait is bounded: after FR_SPIN_LIMIT polls a reader sets the
// error flag and goes on (with wrong results), so the grid always drains; the model reports the flag at its next
// synchronisation.
#include "kx_attn_parts.h"
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_front.h"
#include "kx_gemv_body.h"
#include "kx_hand.h"
#include "kx_lds_copy.h"
#include "kx_math.h"
#include "kx_route.h"
#include "kx_wave.h"

namespace {

using namespace kxg;
using namespace kxh;

constexpr int FR_THREADS = 512;      // 8 waves; in the first step wave w < 7 owns the 512-column slices w and w + 7 of a 7168-wide row
constexpr int FR_ROWS = 9;           // rows of q_a | kv_a a workgroup computes: 6 + 2 (+ 1 for the first 64 workgroups)
constexpr int FR_PART_BYTES = 6144;  // head of the dynamic LDS: 2 KB of slice partials, then the q_a row / the head's q

struct FrontArgs {
  const uint16_t *x, *input_ln;  // residual row, input RMSNorm weights [hidden]
  const uint16_t *w_qkv;         // bf16 [q_rank + kv_rank + rope, hidden]
  const uint16_t *qa_ln, *w_qb;  // q_a RMSNorm weights [q_rank], bf16 [heads * (nope + rope), q_rank]
  QAbsArgs qa;                   // kvb, rope_row, qabs, w_kv_ln, cache, dims, pos
  uint32_t *hand;                // tagged words: [q_rank] q_a, [kv_rank + rope] kv_a, [heads * (nope + rope)] q
  int hidden, q_rank, rows_b;
  float eps;
  uint32_t tag;                  // this launch's tag, in the upper half of every word handed over
  int *err;
};

__global__ void __launch_bounds__(FR_THREADS) attn_front_k(FrontArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t fr_lds[];
  __shared__ float s_ws[4];
  __shared__ float s_scale;
  float *part = (float *)fr_lds;                 // [FR_ROWS][S] of phase A, [rows_b][4] of the q_b step, [8][cq] of the absorb
  uint16_t *s_row = (uint16_t *)(fr_lds + 2048); // the q_a row (q_rank bf16); later the head's q as floats
  uint8_t *big = fr_lds + FR_PART_BYTES;         // the q_b rows of this workgroup
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = blockIdx.x;
  const int H = a.hidden, S = H >> 9, kva = a.qa.kv_rank + a.qa.rope;
  const int rows_a = a.q_rank / (int)gridDim.x;  // 6
  uint32_t *hand_qa = a.hand, *hand_kv = a.hand + a.q_rank, *hand_q = hand_kv + kva;

  // rows of [q_a ; kv_a] this workgroup computes: rows_a of q_a, two of kv_a, and one more of kv_a while they last
  auto row_of = [&](int i) {
    if (i < rows_a) return bid * rows_a + i;
    const int k = i < rows_a + 2 ? 2 * bid + (i - rows_a) : 2 * (int)gridDim.x + bid;
    return k < kva ? a.q_rank + k : -1;
  };

  const int row_bytes = a.q_rank * 2;
  // ---- every load that does not depend on another workgroup goes out now, in the order of need: the row for the
  // RMSNorm, this wave's activations and weights, and behind them the operands of the later steps (the q_a RMSNorm
  // weights of the q_b step, the W_UK block of the absorb), which then lie in registers when their step comes
  uint4 wbuf[FR_ROWS][2], xr[2], gr[2], nx[4], gb[4], wuk_r[16];
  const int s0 = wave, s1 = wave + 7;  // this wave's slices (wave 7 computes nothing in phase A)
  const int SB = a.q_rank >> 9;        // slices of the q_b GEMV: 3 at Kimi-K2 shapes; the launcher allows up to 4
  const int cq = a.qa.kv_rank >> 2, ncg = cq >> 3;  // absorb: columns per workgroup, groups of 8 of them
  const int ab_chain = tid / ncg, ab_cg = tid - ab_chain * ncg;  // absorb item of this thread (tid < 8 * ncg)
  if (tid < 256) {
    const int chunks = H >> 3;
#pragma unroll
    for (int j = 0; j < 4; ++j) nx[j] = ((const uint4 *)a.x)[min(tid + 256 * j, chunks - 1)];
  }
  issue_order();
  if (wave < 7) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const uint32_t col = (uint32_t)(k ? s1 : s0) * 512u + (uint32_t)lane * 8u;
      xr[k] = *(const uint4 *)(a.x + col);
      gr[k] = *(const uint4 *)(a.input_ln + col);
    }
#pragma unroll
    for (int i = 0; i < FR_ROWS; ++i) {
      const int row = max(row_of(i), 0);
#pragma unroll
      for (int k = 0; k < 2; ++k)
        wbuf[i][k] = ld_stream16(a.w_qkv + (size_t)row * H + (uint32_t)(k ? s1 : s0) * 512u + (uint32_t)lane * 8u);
    }
  }
  issue_order();
#pragma unroll
  for (int s = 0; s < 4; ++s)
    if (s < SB) gb[s] = *(const uint4 *)(a.qa_ln + s * 512 + lane * 8);
  if (tid < 8 * ncg) {  // 16 rows of W_UK[h] for this thread's chain and column group (nope = 128: the launcher checks)
    const uint16_t *wuk = a.qa.kvb + (size_t)(bid >> 2) * (a.qa.nope + a.qa.v_head) * a.qa.kv_rank + (bid & 3) * cq + ab_cg * 8;
#pragma unroll
    for (int i = 0; i < 16; ++i) wuk_r[i] = ld_stream16(wuk + (size_t)(ab_chain + 8 * i) * a.qa.kv_rank);
  }
  // input RMSNorm scale: gemv_body's prologue (the first 256 threads own the 8-element chunks t, t + 256, ...)
  {
    const int chunks = H >> 3;
    float v = 0.0f;
    if (tid < 256) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (tid + 256 * j < chunks) {
          float f[8];
          unpack8(f, nx[j]);
#pragma unroll
          for (int e = 0; e < 8; ++e) v = __builtin_fmaf(f[e], f[e], v);
        }
    }
    float vv[1] = {v};
    kxw::reduce<1, 64>(vv, lane);
    if (lane == 0 && wave < 4) s_ws[wave] = vv[0];
    kx_lds_barrier();
    if (tid == 0) s_scale = kx_rsqrtf((((s_ws[0] + s_ws[1]) + s_ws[2]) + s_ws[3]) / (float)H + a.eps);
    kx_lds_barrier();
  }
  if (wave < 7) {
    float xs[2][8];
    const float sc = s_scale;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      float g[8];
      unpack8(xs[k], xr[k]);
      unpack8(g, gr[k]);
#pragma unroll
      for (int e = 0; e < 8; ++e) xs[k][e] = kx_bfround(kx_bfround(xs[k][e] * sc) * g[e]);
    }
    auto dot = [&](const uint4 &w, const float (&x8)[8]) {
      float wf[8];
      unpack8(wf, w);
      float acc = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(wf[e], x8[e], acc);
      return acc;
    };
    float v[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[2 * i] = dot(wbuf[i][0], xs[0]);
      v[2 * i + 1] = dot(wbuf[i][1], xs[1]);
    }
    kxw::reduce<16, 64>(v, lane);
    if (kxw::reduce_writer<16, 64>(lane)) {
#pragma unroll
      for (int j = 0; j < kxw::reduce_out<16, 64>(); ++j) {
        const int idx = kxw::reduce_index<16, 64>(lane, j);
        part[(idx >> 1) * S + ((idx & 1) ? s1 : s0)] = v[j];
      }
    }
    float v2[2] = {dot(wbuf[8][0], xs[0]), dot(wbuf[8][1], xs[1])};
    kxw::reduce<2, 64>(v2, lane);
    if (kxw::reduce_writer<2, 64>(lane)) {
#pragma unroll
      for (int j = 0; j < kxw::reduce_out<2, 64>(); ++j) {
        const int idx = kxw::reduce_index<2, 64>(lane, j);
        part[8 * S + (idx ? s1 : s0)] = v2[j];
      }
    }
  }
  kx_lds_barrier();
  if (tid < FR_ROWS) {  // slices left to right, one rounding, handed over
    const int row = row_of(tid);
    if (row >= 0) {
      const float *p = part + tid * S;
      float y = p[0];
      for (int s = 1; s < S; ++s) y += p[s];
      hand_store(a.hand + row, a.tag, kx_bf16_rne(y));
    }
  }

  // ---- waves 4..7: the q_b rows of this workgroup, global -> LDS, 1 KB per copy instruction.  Not earlier: the copies
  // are needed last, and a wave that is held up issuing them (the memory pipeline is full by now) would hold the
  // workgroup's barriers up with it.
  if (wave >= 4) {
    const int units = a.rows_b * row_bytes >> 10;
    const uint8_t *src = (const uint8_t *)a.w_qb + (size_t)bid * a.rows_b * row_bytes + lane * 16;
    const uint32_t dst = (uint32_t)(uintptr_t)big;
    for (int u = wave - 4; u < units; u += 4) kx_copy16_to_lds(src + (size_t)u * 1024, __builtin_amdgcn_readfirstlane(dst + u * 1024));
  }

  // ---- q_a from every workgroup: its RMSNorm scale (the same prologue schedule) and the row itself into LDS
  {
    const int chunks = a.q_rank >> 3;  // at most 256: one chunk per thread
    float v = 0.0f;
    if (tid < chunks) {
      uint32_t o[4];
      hand_load<8>(hand_qa + tid * 8, a.tag, a.err, o);
      ((uint4 *)s_row)[tid] = make_uint4(o[0], o[1], o[2], o[3]);
      float f[8];
      unpack8(f, make_uint4(o[0], o[1], o[2], o[3]));
#pragma unroll
      for (int e = 0; e < 8; ++e) v = __builtin_fmaf(f[e], f[e], v);
    }
    float vv[1] = {v};
    kxw::reduce<1, 64>(vv, lane);
    if (lane == 0 && wave < 4) s_ws[wave] = vv[0];
    kx_wait_copies<0>();  // waves 4..7: their copies have landed
    __syncthreads();
    if (tid == 0) s_scale = kx_rsqrtf((((s_ws[0] + s_ws[1]) + s_ws[2]) + s_ws[3]) / (float)a.q_rank + a.eps);
    __syncthreads();
  }
  // ---- q rows [rows_b * bid, +rows_b) from LDS
  {
    float xs[4][8];
    const float sc = s_scale;
#pragma unroll
    for (int s = 0; s < 4; ++s)
      if (s < SB) {
        float g[8];
        unpack8(xs[s], *(const uint4 *)(s_row + s * 512 + lane * 8));
        unpack8(g, gb[s]);
#pragma unroll
        for (int e = 0; e < 8; ++e) xs[s][e] = kx_bfround(kx_bfround(xs[s][e] * sc) * g[e]);
      }
    // wave w takes rows w, w + 8, ..., w + 40 (the launcher makes rows_b 48): all their LDS reads first, then the
    // products, then one butterfly for four rows and one for two
    auto dot = [&](int r, int s) {
      float wf[8];
      unpack8(wf, *(const uint4 *)(big + (size_t)r * row_bytes + s * 1024 + lane * 16));
      float acc = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(wf[e], xs[s][e], acc);
      return acc;
    };
    float v[16], v2[8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int s = 0; s < 4; ++s) v[i * 4 + s] = s < SB ? dot(wave + 8 * i, s) : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int s = 0; s < 4; ++s) v2[i * 4 + s] = s < SB ? dot(wave + 8 * (4 + i), s) : 0.0f;
    kxw::reduce<16, 64>(v, lane);
    if (kxw::reduce_writer<16, 64>(lane)) {
#pragma unroll
      for (int j = 0; j < kxw::reduce_out<16, 64>(); ++j) {
        const int idx = kxw::reduce_index<16, 64>(lane, j);
        part[(wave + 8 * (idx >> 2)) * 4 + (idx & 3)] = v[j];
      }
    }
    kxw::reduce<8, 64>(v2, lane);
    if (kxw::reduce_writer<8, 64>(lane)) {
#pragma unroll
      for (int j = 0; j < kxw::reduce_out<8, 64>(); ++j) {
        const int idx = kxw::reduce_index<8, 64>(lane, j);
        part[(wave + 8 * (4 + (idx >> 2))) * 4 + (idx & 3)] = v2[j];
      }
    }
    __syncthreads();
    if (tid < a.rows_b) {
      const float *p = part + tid * 4;
      float y = p[0];
      for (int s = 1; s < SB; ++s) y += p[s];
      hand_store(hand_q + (size_t)bid * a.rows_b + tid, a.tag, kx_bf16_rne(y));
    }
  }
  // ---- workgroup 0: kv_a from everybody -> RMSNorm of the latent part, RoPE of the shared key, the cache row.
  // kxa::kv_finish_block's schedule, with the row taken from the tagged words.
  if (bid == 0) {
    const int kv_rank = a.qa.kv_rank, rope = a.qa.rope, half = rope >> 1, chunks = kv_rank >> 3;
    uint16_t *crow = a.qa.cache + (size_t)a.qa.pos * kva;
    uint4 mine = make_uint4(0, 0, 0, 0);
    float v = 0.0f;
    if (tid < chunks) {  // chunks <= 256 (the launcher checks)
      uint32_t o[4];
      hand_load<8>(hand_kv + tid * 8, a.tag, a.err, o);
      mine = make_uint4(o[0], o[1], o[2], o[3]);
      float f[8];
      unpack8(f, mine);
#pragma unroll
      for (int e = 0; e < 8; ++e) v = __builtin_fmaf(f[e], f[e], v);
    }
    float vv[1] = {v};
    kxw::reduce<1, 64>(vv, lane);
    __syncthreads();
    if (tid < 4) s_ws[tid] = 0.0f;
    __syncthreads();
    if (tid < 256 && lane == 0) s_ws[wave] = vv[0];
    __syncthreads();
    const float scale = kx_rsqrtf((((s_ws[0] + s_ws[1]) + s_ws[2]) + s_ws[3]) / (float)kv_rank + a.qa.eps);
    if (tid < chunks) {
      float f[8], g[8];
      unpack8(f, mine);
      unpack8(g, ((const uint4 *)a.qa.w_kv_ln)[tid]);
      uint32_t o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        o[e] = (uint32_t)kx_bf16_rne(kx_bfround(f[2 * e] * scale) * g[2 * e]) | ((uint32_t)kx_bf16_rne(kx_bfround(f[2 * e + 1] * scale) * g[2 * e + 1]) << 16);
      ((uint4 *)crow)[tid] = make_uint4(o[0], o[1], o[2], o[3]);
    }
    if (tid >= 256 && tid < 256 + (half >> 1)) {  // two interleaved pairs per thread (rope is a multiple of 4)
      uint32_t o[2];
      hand_load<4>(hand_kv + kv_rank + 4 * (tid - 256), a.tag, a.err, o);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int p = 2 * (tid - 256) + u;
        float lo, hi;
        kxa::rope_pair(bf_lo(o[u]), bf_hi(o[u]), kx_bf16_f32(a.qa.rope_row[p]), kx_bf16_f32(a.qa.rope_row[half + p]), lo, hi);
        crow[kv_rank + p] = kx_bf16_rne(lo);
        crow[kv_rank + half + p] = kx_bf16_rne(hi);
      }
    }
  }
  // ---- a quarter of the head's q_abs: the sums of kxa::absorb_head_block for columns [cq * j, cq * (j + 1))
  {
    const int nope = a.qa.nope, rope = a.qa.rope, kv_rank = a.qa.kv_rank, qk = nope + rope, half = rope >> 1;
    const int h = bid >> 2, j = bid & 3;
    float *ab_part = (float *)big;     // [8][cq]: the q_b rows are spent
    float *qs = (float *)s_row;        // [qk]
    float *out = a.qa.qabs + (size_t)h * (kv_rank + rope);
    __syncthreads();  // s_row (the q_a row) and the q_b rows are no longer read
    if (tid < (qk >> 2)) {
      uint32_t o[2];
      hand_load<4>(hand_q + (size_t)h * qk + tid * 4, a.tag, a.err, o);
      qs[tid * 4 + 0] = bf_lo(o[0]); qs[tid * 4 + 1] = bf_hi(o[0]);
      qs[tid * 4 + 2] = bf_lo(o[1]); qs[tid * 4 + 3] = bf_hi(o[1]);
    }
    __syncthreads();
    if (tid < 8 * ncg) {  // chain ab_chain over d = ab_chain, ab_chain + 8, ..., W_UK rows from the registers
      float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float wf[8];
        unpack8(wf, wuk_r[i]);
        const float qd = qs[ab_chain + 8 * i];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(wf[e], qd, acc[e]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ab_part[ab_chain * cq + ab_cg * 8 + e] = acc[e];
    }
    __syncthreads();
    for (int c = tid; c < cq; c += FR_THREADS) {
      const float *p = ab_part + c;
      const float s = ((p[0] + p[cq]) + (p[2 * cq] + p[3 * cq])) + ((p[4 * cq] + p[5 * cq]) + (p[6 * cq] + p[7 * cq]));
      out[j * cq + c] = kx_bfround(s);
    }
    if (j == 3 && tid < half) {
      float lo, hi;
      kxa::rope_pair(qs[nope + 2 * tid], qs[nope + 2 * tid + 1], kx_bf16_f32(a.qa.rope_row[tid]), kx_bf16_f32(a.qa.rope_row[half + tid]),
                     lo, hi);
      out[kv_rank + tid] = lo;
      out[kv_rank + half + tid] = hi;
    }
  }
}


// ---------------------------------------------------------------------------------------------------------------
// The back of the attention block for one token as one launch: the merge of the attention's span partials, the
// per-head W_UV product (src/kimi_exec.cu:818 as W_UV) and o_proj with the residual add (:826-827).  As launches
// of their own (the W_UV GEMV that merges while it loads, the o_proj GEMV) the second one streams 117 MB and
// cannot ask for a byte of it before the first has drained.  Here every workgroup merges and multiplies its quarter
// of a head, hands the 32 values over as tagged words, requests the first five tiles of its o_proj rows and then
// takes all 8192 values from the other workgroups.  A wave's loads return in order, so its polls come back behind
// the weights it has asked for -- which is when the others have handed over, about: five of a workgroup's seven
// tiles are in registers by then.  The tiles are not requested before the hand-over: a CU's memory pipeline takes
// requests in order, and the 32 stores would sit behind 160 KB of them (measured: 2.5 us later, no gain from the
// earlier start).  Sums as in kx_gemv_body.h (lane partial over 8 columns, butterfly over the wave, slices left to
// right) and in its merge of the partials: equal to the separate launches to the bit.
constexpr int BK_THREADS = 512;  // 8 waves: wave w owns rows 4 w .. of its quarter head, then the slices w and w + 8 of o_proj
constexpr int BK_PRE = 5;        // o_proj tiles (4 rows x 2 slices per wave) in flight per wave
constexpr int BK_SPANS = 32;     // span partials a thread holds in registers

struct BackArgs {
  const float *pm, *pz, *po;  // attention partials of the token: [spans][heads], same, [spans][heads][kv_rank]
  int spans, heads;
  const uint16_t *kvb;        // kv_b: W_UV[h] = rows h * (nope + v_head) + nope .. of it
  int nope, v_head, kv_rank;
  const uint16_t *w_o;        // bf16 [hidden, heads * v_head]
  uint16_t *x;                // the residual row, updated in place
  int hidden, vd;
  uint32_t *hand;             // tagged words: [heads * v_head] attention output; HEAD: [hidden] residual row, [2 * experts] router logits
  uint32_t tag;
  int *err;
  KxMoeHeadArgs hd;           // HEAD only
};

constexpr int HD_TILES = 5;   // the head's rows as tiles of 4: 8 gate, 8 up, 2 router rows, 2 unused
constexpr int HD_O_TILES = 7; // o_proj tiles of a workgroup when the head rides along (hidden = 28 * 256)

// HEAD: the launch goes on with the head of the MoE layer (the router and shared gate/up launch of kx_moe.hip):
// post-attention RMSNorm, the shared expert's gate and up rows with SwiGLU, the router's logits, top-k and bucketing.
// The residual row travels between the workgroups as the attention output does; a workgroup's 18 rows of the three
// matrices are requested into the o_proj tiles' registers as those are used up, so the weight stream does not stop
// for the hand-over.  The last workgroup takes the logits from the others and routes (kx_route.h, the same code the
// router launch runs).  Sums as in kx_gemv_body.h.
template <bool HEAD>
__global__ void __launch_bounds__(BK_THREADS) attn_back_k(BackArgs a) {
  __shared__ float s_x[512];                                   // the head's merged attention output, bf16 values
  __shared__ __attribute__((aligned(16))) uint16_t s_att[8192];  // the token's attention output, all heads
  __shared__ float s_part[8 * 4 * 16];                         // [row of the workgroup][slice]
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = blockIdx.x, h = bid >> 2, jq = bid & 3;
  const int rows_o = a.hidden / (int)gridDim.x, tiles = HEAD ? HD_O_TILES : rows_o >> 2;  // 28 rows, 7 tiles of 4 at Kimi-K2 shapes
  const int s0 = wave, s1 = wave + 8;
  // the residual value this thread will add to (a load at that point would come back behind every weight request)
  uint16_t x_old = 0;
  uint4 hd_g[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};  // HEAD: post-attention RMSNorm weights of this lane's columns
  if (tid < rows_o) x_old = a.x[(size_t)bid * rows_o + tid];
  __shared__ float s_logits[HEAD ? 512 : 1], s_bias[HEAD ? 512 : 1];  // the routing workgroup's: one thread per expert
  __shared__ int s_cnt[HEAD ? BK_THREADS : 1], s_act[HEAD ? BK_THREADS : 1];
  __shared__ uint4 s_ids4[4];
  if (HEAD) {
    hd_g[0] = *(const uint4 *)(a.hd.post_ln + s0 * 512 + lane * 8);
    if (s1 * 512 < a.hidden) hd_g[1] = *(const uint4 *)(a.hd.post_ln + s1 * 512 + lane * 8);
    float b = 0.0f;  // the router bias, for the workgroup that routes: in LDS long before it is needed
    if (bid == (int)gridDim.x - 1 && tid < a.hd.experts) b = a.hd.bias[tid];
    s_bias[tid] = b;
  }
  // ---- requests, in the order of need: the head's partials, this wave's W_UV rows
  const size_t my = (size_t)min(lane, a.spans - 1) * a.heads + h;
  const float mj = a.pm[my], zj = a.pz[my];
  float o[BK_SPANS];
#pragma unroll
  for (int j = 0; j < BK_SPANS; ++j) o[j] = j < a.spans ? a.po[((size_t)j * a.heads + h) * a.kv_rank + tid] : 0.0f;
  issue_order();
  uint4 wuv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    wuv[i] = ld_stream16(a.kvb + ((size_t)h * (a.nope + a.v_head) + a.nope + jq * 32 + wave * 4 + i) * a.kv_rank + lane * 8);
  issue_order();
  uint4 wo[BK_PRE][4][2];
  const uint16_t *wo_base = a.w_o + (size_t)bid * rows_o * a.vd + lane * 8;
  auto load_tile = [&](uint4 (&buf)[4][2], int t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      buf[i][0] = ld_stream16(wo_base + (size_t)(t * 4 + i) * a.vd + s0 * 512);
      buf[i][1] = ld_stream16(wo_base + (size_t)(t * 4 + i) * a.vd + s1 * 512);
    }
  };
  // ---- the merge of the span partials (kx_gemv_body.h load_x): M = max M_j; w_j = exp(M_j - M);
  // Z = fma(Z_j, w_j, Z), O = fma(O_j, w_j, O) over the spans in order; x = bf(O / Z).  Thread c owns column c.
  {
    const float M = kxw::wave_max_f32(lane < a.spans ? mj : -__builtin_inff());
    const float wj = kx_expf(mj - M);
    float Z = 0.0f, O = 0.0f;
    for (int j = 0; j < a.spans; ++j)
      Z = __builtin_fmaf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, zj), j)),
                         __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), j)), Z);
#pragma unroll
    for (int j = 0; j < BK_SPANS; ++j)
      if (j < a.spans) O = __builtin_fmaf(o[j], __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), j)), O);
    s_x[tid] = kx_bfround(O / Z);
  }
  kx_lds_barrier();
  // ---- W_UV: rows 32 jq + 4 wave + i of the head; one 512-column slice, so the butterfly's value is the row's
  {
    float xs[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) xs[e] = s_x[lane * 8 + e];
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float wf[8];
      unpack8(wf, wuv[i]);
      float acc = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(wf[e], xs[e], acc);
      v[i] = acc;
    }
    kxw::reduce<4, 64>(v, lane);
    if (kxw::reduce_writer<4, 64>(lane)) {
#pragma unroll
      for (int j = 0; j < kxw::reduce_out<4, 64>(); ++j) {
        const int i = kxw::reduce_index<4, 64>(lane, j);
        hand_store(a.hand + (size_t)h * a.v_head + jq * 32 + wave * 4 + i, a.tag, kx_bf16_rne(v[j]));
      }
    }
  }
  // ---- the first o_proj tiles, behind the hand-over and in front of the polls
#pragma unroll
  for (int t = 0; t < BK_PRE; ++t) load_tile(wo[t], min(t, tiles - 1));
  issue_order();
  // ---- all of the token's attention output: 8192 words = 2048 requests of 16 bytes, four per thread; request i of
  // thread t is number 512 i + t, so that a wave's request covers 1 KB in a row.  Asked for again until every word
  // carries the tag.
  {
    const uint32_t *src = a.hand + (size_t)tid * 4;
    hand4 v[4];
    int polls = 0;
    while (true) {
#pragma unroll
      for (int i = 0; i < 4; ++i) hand_request4(src + (size_t)i * 2048, v[i]);
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3])::"memory");
      if ((hand_tagged(v[0], a.tag) && hand_tagged(v[1], a.tag) && hand_tagged(v[2], a.tag) && hand_tagged(v[3], a.tag)) || hand_give_up(polls, a.err)) break;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) ((uint2 *)s_att)[i * 512 + tid] = hand_pack(v[i]);
  }
  kx_lds_barrier();
  // ---- o_proj rows [rows_o * bid, +rows_o): BK_PRE tiles in flight, a tile's registers take the tile BK_PRE further on
  float xo[2][8];
  unpack8(xo[0], *(const uint4 *)(s_att + s0 * 512 + lane * 8));
  unpack8(xo[1], *(const uint4 *)(s_att + s1 * 512 + lane * 8));
  auto compute_tile = [&](const uint4 (&buf)[4][2], int t) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        float wf[8];
        unpack8(wf, buf[i][k]);
        float acc = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(wf[e], xo[k][e], acc);
        v[i * 2 + k] = acc;
      }
    kxw::reduce<8, 64>(v, lane);
    if (kxw::reduce_writer<8, 64>(lane)) {
#pragma unroll
      for (int j = 0; j < kxw::reduce_out<8, 64>(); ++j) {
        const int idx = kxw::reduce_index<8, 64>(lane, j);
        s_part[(t * 4 + (idx >> 1)) * 16 + ((idx & 1) ? s1 : s0)] = v[j];
      }
    }
  };
  // HEAD: row r of the workgroup's head tiles -> the weight row it stands for (nullptr: none).  Tile 0 comes first in
  // every sense: two router rows (the first experts / 2 workgroups), or a gate and an up row of the eight shared rows
  // that the last workgroup, which routes instead, leaves to the eight workgroups behind the router's; then the
  // workgroup's eight gate rows and eight up rows.
  const int E = a.hd.experts, last = (int)gridDim.x - 1;
  const int extra = HEAD && bid >= (E >> 1) && bid < (E >> 1) + 8 ? 8 * last + bid - (E >> 1) : -1;  // shared row taken over
  auto head_row = [&](int r) -> const uint16_t * {
    if (bid == last) return nullptr;
    if (r < 2) return 2 * bid < E ? a.hd.w_router + (size_t)(2 * bid + r) * a.hidden : nullptr;
    if (r < 4) return extra >= 0 ? (r == 2 ? a.hd.w_gate : a.hd.w_up) + (size_t)extra * a.hidden : nullptr;
    if (r < 12) return a.hd.w_gate + (size_t)(8 * bid + r - 4) * a.hidden;
    return a.hd.w_up + (size_t)(8 * bid + r - 12) * a.hidden;
  };
  auto load_head_tile = [&](uint4 (&buf)[4][2], int j) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint16_t *row = head_row(4 * j + i);
      buf[i][0] = buf[i][1] = make_uint4(0, 0, 0, 0);
      if (row) {
        buf[i][0] = ld_stream16(row + s0 * 512 + lane * 8);
        if (s1 * 512 < a.hidden) buf[i][1] = ld_stream16(row + s1 * 512 + lane * 8);
      }
    }
  };
  if constexpr (HEAD) {
#pragma unroll
    for (int t = 0; t < HD_O_TILES; ++t) {
      compute_tile(wo[t % BK_PRE], t);
      if (t + BK_PRE < HD_O_TILES) load_tile(wo[t % BK_PRE], t + BK_PRE);
      else load_head_tile(wo[t % BK_PRE], t + BK_PRE - HD_O_TILES);  // head tile j lies in wo[(HD_O_TILES + j) % BK_PRE]
    }
  } else {
    for (int t0 = 0; t0 < tiles; t0 += BK_PRE) {
#pragma unroll
      for (int u = 0; u < BK_PRE; ++u) {
        const int t = t0 + u;
        if (t < tiles) {
          compute_tile(wo[u], t);
          if (t + BK_PRE < tiles) load_tile(wo[u], t + BK_PRE);
        }
      }
    }
  }
  kx_lds_barrier();
  // ---- slices left to right, then x = bf(x + bf(y))  (add_k, :248-251)
  uint32_t *hand_x = a.hand + (size_t)a.heads * a.v_head;
  if (tid < rows_o) {
    const float *p = s_part + tid * 16;
    float y = p[0];
#pragma unroll
    for (int s = 1; s < 16; ++s) y += p[s];
    const uint16_t x_new = kx_bf16_rne(kx_bf16_f32(x_old) + kx_bfround(y));
    a.x[(size_t)bid * rows_o + tid] = x_new;
    if (HEAD) hand_store(hand_x + (size_t)bid * rows_o + tid, a.tag, x_new);
  }
  if constexpr (!HEAD) return;
  // ================================================================ the head of the MoE layer
  const int H = a.hidden, S = H >> 9;
  uint16_t *s_xrow = s_att;  // the residual row; the attention output is spent
  __shared__ float s_ws[4];
  __shared__ float s_scale;
  uint32_t *hand_lg = hand_x + H;
  if (bid == last) {
    // ---- the last workgroup routes: logits from the tagged words into LDS (the bias lies there since the start),
    // then kx_route.h
    if (tid < (E >> 1)) {  // two logits = four words
      uint32_t o[2];
      hand_load<4>(hand_lg + tid * 4, a.tag, a.err, o);
      s_logits[2 * tid] = __builtin_bit_cast(float, o[0]);
      s_logits[2 * tid + 1] = __builtin_bit_cast(float, o[1]);
    }
    __syncthreads();
    kxr::route_block_any<false>(s_logits, s_bias, a.hd.ids, a.hd.weights, 1, E, a.hd.topk, a.hd.routed_scale, a.hd.counts, a.hd.offsets,
                                a.hd.pairs, a.hd.work, a.hd.n_active, s_ids4, s_cnt, s_act, nullptr);
    return;
  }
  {  // the residual row from every workgroup: H / 4 requests of 16 bytes, request i of thread t is number 512 i + t
    const uint32_t *src = hand_x + (size_t)tid * 4;
    const int nreq = H >> 2;
    // The last request is made by half of the threads only.  A request under a condition gives the registers it fills a
    // second definition, which leaves the compiler free to move them between the request and the wait, while the load
    // is on its way; in this loop it does not (a variant of the front launch where it did never found its tags and
    // ended in the error flag: the failure is loud).  Asking for a duplicate instead costs 0.8 % of the decode rate.
    hand4 v[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    int polls = 0;
    while (true) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (i * 512 + tid < nreq) hand_request4(src + (size_t)i * 2048, v[i]);
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3])::"memory");
      bool ok = true;
#pragma unroll
      for (int i = 0; i < 4; ++i) ok = ok && (i * 512 + tid >= nreq || hand_tagged(v[i], a.tag));
      if (ok || hand_give_up(polls, a.err)) break;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i * 512 + tid < nreq) ((uint2 *)s_xrow)[i * 512 + tid] = hand_pack(v[i]);
  }
  __syncthreads();  // every request of this kernel has landed by now
  {  // the row's RMSNorm scale: gemv_body's prologue (the first 256 threads own the 8-element chunks t, t + 256, ...)
    const int chunks = H >> 3;
    float v = 0.0f;
    if (tid < 256)
      for (int c = tid; c < chunks; c += 256) {
        float f[8];
        unpack8(f, ((const uint4 *)s_xrow)[c]);
#pragma unroll
        for (int e = 0; e < 8; ++e) v = __builtin_fmaf(f[e], f[e], v);
      }
    float vv[1] = {v};
    kxw::reduce<1, 64>(vv, lane);
    if (lane == 0 && wave < 4) s_ws[wave] = vv[0];
    __syncthreads();
    if (tid == 0) s_scale = kx_rsqrtf((((s_ws[0] + s_ws[1]) + s_ws[2]) + s_ws[3]) / (float)H + a.hd.eps);
    __syncthreads();
  }
  const float sc = s_scale;
  auto normed8 = [&](float (&o)[8], uint4 raw, uint4 g8) {
    float g[8];
    unpack8(o, raw);
    unpack8(g, g8);
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = kx_bfround(kx_bfround(o[e] * sc) * g[e]);
  };
  float xh[2][8];
  normed8(xh[0], *(const uint4 *)(s_xrow + s0 * 512 + lane * 8), hd_g[0]);
  normed8(xh[1], *(const uint4 *)(s_xrow + min(s1, S - 1) * 512 + lane * 8), hd_g[1]);
  auto head_tile = [&](const uint4 (&buf)[4][2], int j) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        float wf[8];
        unpack8(wf, buf[i][k]);
        float acc = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(wf[e], xh[k][e], acc);
        v[i * 2 + k] = acc;
      }
    kxw::reduce<8, 64>(v, lane);
    if (kxw::reduce_writer<8, 64>(lane)) {
#pragma unroll
      for (int q = 0; q < kxw::reduce_out<8, 64>(); ++q) {
        const int idx = kxw::reduce_index<8, 64>(lane, q);
        if (!(idx & 1) || s1 < S) s_part[(j * 4 + (idx >> 1)) * 16 + ((idx & 1) ? s1 : s0)] = v[q];
      }
    }
  };
  auto slice_sum = [&](int r) {
    const float *p = s_part + r * 16;
    float y = p[0];
    for (int q = 1; q < S; ++q) y += p[q];
    return y;
  };
  // ---- tile 0 first and on its own: the router's logits are what the last workgroup waits for
  const bool tile0 = 2 * bid < E || extra >= 0;
  if (tile0) {
    head_tile(wo[HD_O_TILES % BK_PRE], 0);
    __syncthreads();
    if (tid < 2 && 2 * bid < E) {  // a router logit: fp32 (KX_EPI_F32), handed over as two tagged halves
      const int e = 2 * bid + tid;
      const float y = slice_sum(tid);
      const uint32_t u = __builtin_bit_cast(uint32_t, y);
      hand_store(hand_lg + 2 * e, a.tag, (uint16_t)(u & 0xffffu));
      hand_store(hand_lg + 2 * e + 1, a.tag, (uint16_t)(u >> 16));
      a.hd.logits[e] = y;
    }
  }
  // the normed row for the routed experts' launch: 8 chunks of 8 values by each of the first workgroups
  if (tid >= 64 && tid < 72 && 8 * bid + tid - 64 < (H >> 3)) {
    const int c = 8 * bid + tid - 64;
    float f[8];
    normed8(f, ((const uint4 *)s_xrow)[c], ((const uint4 *)a.hd.post_ln)[c]);
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (uint32_t)kx_bf16_rne(f[2 * e]) | ((uint32_t)kx_bf16_rne(f[2 * e + 1]) << 16);
    ((uint4 *)a.hd.n_out)[c] = make_uint4(o[0], o[1], o[2], o[3]);
  }
#pragma unroll
  for (int j = 1; j < HD_TILES; ++j) head_tile(wo[(HD_O_TILES + j) % BK_PRE], j);
  __syncthreads();
  // KX_EPI_SWIGLU: rows 4 + t (gate) and 12 + t (up) of the tiles; the row taken over from the last workgroup: 2 and 3
  if (tid < 8) a.hd.smid[8 * bid + tid] = kx_bf16_rne(kx_swiglu(kx_bfround(slice_sum(4 + tid)), kx_bfround(slice_sum(12 + tid))));
  if (tid == 8 && extra >= 0) a.hd.smid[extra] = kx_bf16_rne(kx_swiglu(kx_bfround(slice_sum(2)), kx_bfround(slice_sum(3))));
}

}  // namespace

// g_qkv: the q_a | kv_a GEMV as the separate launch would get it (w0 = [q_rank + kv_rank + rope, hidden], x = the
// residual row, norm_w = the input RMSNorm weights); g_qb: the q_b GEMV (w0 = [heads * (nope + rope), q_rank],
// norm_w = the q_a RMSNorm weights).  hand: (q_rank + kv_rank + rope + heads * (nope + rope)) words of device memory;
// tag: a value in [1, 65535] that differs from the previous launch's on the same `hand`; err: one int, zero until a
// wait of some launch gave up.  *done = false, nothing launched, when the shapes or the device do not allow the
// fused form.  The q_a | kv_a and q rows are not written to g_qkv.out / g_qb.out: nothing after this launch reads them.
int kx_attn_front_launch(const KxGemvArgs &g_qkv, const KxGemvArgs &g_qb, const QAbsArgs &q, uint32_t *hand, uint32_t tag, int *err,
                         bool *done, hipStream_t st) {
  *done = false;
  const int cus = kx_device_cus();  // 0 (query failed): the resident form is declined below
  const int hidden = g_qkv.cols, q_rank = g_qb.cols, qk = q.nope + q.rope, G = 4 * q.heads, kva = q.kv_rank + q.rope;
  if (g_qkv.tokens != 1 || g_qb.tokens != 1 || !hand || !err || !q.cache || !g_qkv.norm_w || !g_qb.norm_w || tag < 1 || tag > 65535) return KX_OK;
  if (G > cus || hidden != 14 * 512 || q_rank % 512 || q_rank / 512 > 4 || q_rank / 8 > 256) return KX_OK;
  if (g_qkv.rows != q_rank + kva || g_qb.rows != q.heads * qk || qk % 16 || q.rope % 4 || q.kv_rank % 4 || q.rope / 2 > 256 || qk / 4 > FR_THREADS) return KX_OK;
  const int rows_a = q_rank / G, rows_b = qk / 4;
  if (rows_b != 48 || q.nope != 128 || q.kv_rank / 4 > FR_THREADS || q_rank % G || rows_a != FR_ROWS - 3 || kva < 2 * G || kva > 3 * G || q.kv_rank % 32 || q.kv_rank / 8 > 256) return KX_OK;
  const size_t qb_bytes = (size_t)rows_b * q_rank * 2;
  if (qb_bytes % 1024 || (size_t)rows_b * 16 > 2048 || (size_t)FR_ROWS * 14 * 4 > 2048 || (size_t)q_rank * 2 > FR_PART_BYTES - 2048 ||
      (size_t)qk * 4 > FR_PART_BYTES - 2048 || qb_bytes < (size_t)8 * (q.kv_rank / 4) * 4)
    return KX_OK;
  const size_t lds = FR_PART_BYTES + qb_bytes;
  if (lds > 156 * 1024) return KX_OK;
  static bool attr_set = false;
  if (!attr_set) {
    KX_HIP(hipFuncSetAttribute((const void *)attn_front_k, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
    attr_set = true;
  }
  FrontArgs a = {};
  a.x = g_qkv.x; a.input_ln = g_qkv.norm_w; a.w_qkv = g_qkv.w0; a.qa_ln = g_qb.norm_w; a.w_qb = g_qb.w0;
  a.qa = q;
  a.hand = hand; a.hidden = hidden; a.q_rank = q_rank; a.rows_b = rows_b; a.eps = g_qkv.norm_eps; a.tag = tag; a.err = err;
  hipLaunchKernelGGL(attn_front_k, dim3(G), dim3(FR_THREADS), lds, st, a);
  KX_LAUNCH_CHECK();
  *done = true;
  return KX_OK;
}

// The W_UV GEMV that merges the attention partials (g_uv: mla_* set, row_block = v_head) and the o_proj GEMV with the
// residual add (g_o: w0 = [hidden, heads * v_head], out = the residual row) of one token as one launch.  hand:
// kx_back_hand_words words; tag and err as for kx_attn_front_launch.  The W_UV output row (g_uv.out) is not written.
// head: the head of the MoE layer that follows (post-attention norm, shared gate/up, router, routing), taken along
// when its shapes fit the launch's workgroups; *head_done says so.
int kx_attn_back_launch(const KxGemvArgs &g_uv, const KxGemvArgs &g_o, const KxMoeHeadArgs *head, uint32_t *hand, uint32_t tag, int *err,
                        bool *done, bool *head_done, hipStream_t st) {
  *done = false;
  *head_done = false;
  const int cus = kx_device_cus();  // 0 (query failed): the resident form is declined below
  const int heads = g_uv.mla_heads, G = 4 * heads;
  if (g_uv.tokens != 1 || g_o.tokens != 1 || !g_uv.mla_po || !hand || !err || tag < 1 || tag > 65535) return KX_OK;
  if (g_uv.mla_spans < 1 || g_uv.mla_spans > BK_SPANS || G > cus || g_uv.cols != 512 || g_uv.row_block != 128 || g_uv.rows != heads * 128) return KX_OK;
  if (g_o.cols != g_uv.rows || g_o.cols != 16 * 512 || g_o.rows % G || (g_o.rows / G) % 4 || g_o.rows / G > 32 || g_o.rows / G < 4 * BK_PRE || g_o.norm_w) return KX_OK;
  BackArgs a = {};
  a.pm = g_uv.mla_pm; a.pz = g_uv.mla_pz; a.po = g_uv.mla_po; a.spans = g_uv.mla_spans; a.heads = heads;
  a.kvb = g_uv.w0; a.nope = g_uv.w_block_off; a.v_head = g_uv.row_block; a.kv_rank = g_uv.cols;
  if (g_uv.w_block_stride != a.nope + a.v_head) return KX_OK;
  a.w_o = g_o.w0; a.x = (uint16_t *)g_o.out; a.hidden = g_o.rows; a.vd = g_o.cols;
  a.hand = hand; a.tag = tag; a.err = err;
  // the head: 8 gate and 8 up rows and up to 2 router rows per workgroup, columns as 512-wide slices over 8 waves x 2,
  // one thread per expert in the routing; the last workgroup routes, and the 8 workgroups behind the router's take
  // a gate and an up row each for it
  const bool with_head = head && g_o.rows / G == 4 * HD_O_TILES && head->shared_inter == 8 * G && g_o.rows % 512 == 0 && g_o.rows / 512 <= 16 &&
                         g_o.rows <= 8192 && head->experts % 2 == 0 && head->experts / 2 + 8 < G && head->experts <= 512 &&
                         head->topk >= 1 && head->topk <= 32 && head->topk <= head->experts && g_o.rows / 8 >= 1 && g_o.rows / 64 <= G;
  if (with_head) {
    a.hd = *head;
    hipLaunchKernelGGL(attn_back_k<true>, dim3(G), dim3(BK_THREADS), 0, st, a);
  } else {
    hipLaunchKernelGGL(attn_back_k<false>, dim3(G), dim3(BK_THREADS), 0, st, a);
  }
  KX_LAUNCH_CHECK();
  *done = true;
  *head_done = with_head;
  return KX_OK;
}
