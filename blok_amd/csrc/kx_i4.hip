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
//    (16,8,4,2,1; see kx_wave.h), then a sequential sum over the 1024-column slices.
//
// All arithmetic is IEEE binary32 (fma, mul, add), so a scalar host program
// that follows the same order reproduces the result bit for bit.
#include "kx_arrive.h"
#include "kx_hand.h"
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_gemv_body.h"
#include "kx_math.h"
#include "kx_wave.h"

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

__device__ __forceinline__ void prep_xgroup(XGroup &g, const uint4 (&raw)[4] /* 32 bf16 of the group */) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint4 u = raw[w];  // x[8w .. 8w+7]
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

struct I4Args {
  const uint32_t *packed0;
  const uint16_t *scale0;
  const uint32_t *packed1;  // DUAL only
  const uint16_t *scale1;
  const uint16_t *x;  // bf16 rows of `cols`
  uint16_t *out;      // bf16 rows of `rows`, indexed by pair
  const int4 *work;   // {expert, first, last, pairs[first]} per expert with work, then {-1,..};
                      // nullptr: one matrix, pairs 0..n_pairs-1
  const int *pairs;   // pair ids sorted by expert
  int n_pairs;        // used when work == nullptr
  int n_slots;        // records in `work`
  int rows, cols;
  int x_div;   // activation row = pair / x_div
  int ks, rs;  // 1024-column slices, row sets; ks*rs waves per workgroup
  int nt;      // tiles per chunk
  size_t expert_words, expert_scales;
  int cnt_lo, cnt_hi;  // only experts with cnt_lo <= pairs <= cnt_hi are processed by this launch
  KxMoeTail tail;      // tail.counter != nullptr: single-matrix launches finish the MoE layer (see moe_tail_arrive)
  uint32_t *hand;      // HAND: the gate/up outputs as tagged words [pair][rows] (kx_hand.h), written (1) or read as activations (2)
  uint32_t tag;
  int *err;
};

constexpr int I4_RI = 2;  // rows per half-wave per tile

// Rows of a chunk for tiles of rt rows: 32 for the fused gate/up kernel; for one matrix 112 when rt divides it
// (7168 rows / 112 = 64 chunks per expert: 8 experts fill the 512 resident workgroups exactly once), else 64.
__host__ __device__ constexpr int i4_chunk_rows(bool dual, int rt) { return dual ? 32 : (112 % rt == 0 ? 112 : 64); }

// Called by every thread of a workgroup that has finished its contributions to the MoE layer's down projection: a
// routed expert's chunk inside row block blk_a and/or a chunk of the shared expert's down GEMV inside row block
// blk_b (-1: none), blocks of `block_rows` rows.  The outputs were stored with device-scope stores; the workgroup
// counts itself in on the counters of its blocks, and where it completes a block -- n_active experts and
// shared_chunks shared chunks -- it combines it: down = bf(sum_slot y_slot * w_slot) in slot order,
// down = bf(down + bf(shared)), x = bf(x + down).  Nothing waits for another workgroup.  Counters are left at zero.
__device__ __forceinline__ void moe_tail_arrive(const KxMoeTail &t, int blk_a, int blk_b, int block_rows, int rows,
                                                const uint16_t *eout) {
  __shared__ int s_last[2];
  kx_arrive_writes_done();
  __syncthreads();  // every lane's outputs lie before the counting lanes' release (kx_arrive.h)
  if (threadIdx.x < 2) {
    const int blk = threadIdx.x ? blk_b : blk_a;
    int last = 0;
    if (blk >= 0) last = kx_arrive_is_last(t.counter + blk, *t.n_active + t.shared_chunks);
    s_last[threadIdx.x] = last;
  }
  __syncthreads();
  for (int which = 0; which < 2; ++which) {
    if (!s_last[which]) continue;
    const int blk = which ? blk_b : blk_a;
    const int r0 = blk * block_rows;
    for (int idx = threadIdx.x; idx < block_rows * t.tokens; idx += blockDim.x) {
      const int rc = idx % block_rows, tok = idx / block_rows, row = r0 + rc;
      const uint16_t *y = eout + (size_t)tok * t.topk * rows + row;
      const float *w = t.route_w + (size_t)tok * t.topk;
      const uint16_t sh = kx_arrive_load(t.sy + (size_t)tok * rows + row);
      float acc = 0.0f;
      int k = 0;
      for (; k + 8 <= t.topk; k += 8) {  // the loads of eight slots go out together; the sum stays in slot order
        uint16_t v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = kx_arrive_load(y + (size_t)(k + j) * rows);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc = __builtin_fmaf(kx_bf16_f32(v[j]), w[k + j], acc);
      }
      for (; k < t.topk; ++k)
        acc = __builtin_fmaf(kx_bf16_f32(kx_arrive_load(y + (size_t)k * rows)), w[k], acc);
      const float down = kx_bfround(kx_bfround(acc) + kx_bf16_f32(sh));
      uint16_t *xr = t.x + (size_t)tok * t.x_stride + row;
      *xr = (t.flags & 1u) ? kx_bf16_rne(down) : kx_bf16_rne(kx_bf16_f32(*xr) + down);
    }
    if (threadIdx.x == 0) kx_arrive_reset(t.counter + blk);
  }
}

// A workgroup of ks*rs waves takes chunks of nt tiles of RT = rs*4 rows of one expert.
// Wave (s, rset): slice s of rows rset*4 .. rset*4+3 of each tile; its half-waves take
// alternate rows.  Per chunk: the group scales of all its rows are copied into LDS (global ->
// LDS loads, no registers), the packed words stream through two register buffers (tile i+1
// is in flight while tile i is computed), partial sums go to LDS and are summed over the
// slices at the end of the chunk.  While a chunk is computed the next one is prepared: its
// work record is read and its scales are copied into the second scale buffer at the start;
// the first tile and activations of whatever comes next (a further pass, the next chunk) are requested before the epilogue.  A last chunk that would
// run past the matrix is moved back to end at the last row (the overlap is computed twice,
// with identical results, and written once).
// KS_T > 0 fixes ks (and rs, nt) at compile time; 0 reads them from the arguments.
// FILTER: the launch processes only the experts whose pair count lies in [cnt_lo, cnt_hi]
// `idle` is called once, where the last chunk's loads have landed and nothing more will be requested: what it
// requests arrives during the epilogue.
// HAND (one token, one chunk per workgroup, inside a launch whose workgroups are all resident): 1 = every output is
// also handed over as a tagged word, and the workgroup may have more waves than the chunk shape uses (they keep the
// barriers); 2 = the activations are not read from a.x but collected from the tagged words of the pair's row, one
// 16-byte request per thread (4 * blockDim.x = cols), through LDS.
template <bool DUAL, int TT, int KS_T, bool FILTER, int CM = 1, int HAND = 0, class Idle>
__device__ __forceinline__ void i4_body(const I4Args &a, const int bid, const int nblocks, float *lds, Idle &&idle) {
  constexpr int MATS = DUAL ? 2 : 1;
  constexpr int RI = I4_RI;
  constexpr int NV = RI * MATS * TT;
  constexpr int NOUT = kxw::reduce_out<NV, 32>();
  const int ks = KS_T ? KS_T : a.ks;
  const int rs = KS_T ? (KS_T >= 5 ? 1 : 8 / KS_T) : a.rs;
  const int RT = rs * 2 * RI;
  const int nt = KS_T ? CM * (i4_chunk_rows(DUAL, KS_T >= 5 ? 4 : 32 / KS_T) / (KS_T >= 5 ? 4 : 32 / KS_T)) : a.nt;  // CM: chunks of CM times the rows
  const int CR = RT * nt;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l = lane & 31, h = lane >> 5;
  const int s = wave % ks, rset = wave / ks;
  const bool active = HAND == 1 ? wave < ks * rs : true;
  const int groups = ks * 32, row_words = ks * 128;
  const int n16 = CR * groups / 8;                                // 16-byte pieces of one matrix's chunk scales
  const int sc_pieces = (MATS * n16 + 63) & ~63;                  // per buffer, whole 1 KB runs
  float *part = lds;                                              // [mats][CR][TT][ks]
  uint4 *sc_base = (uint4 *)(lds + ((MATS * CR * TT * ks + 3) & ~3));  // 2 x [mats][CR][groups] bf16
  uint16_t *s_xh = (uint16_t *)(sc_base + 2 * sc_pieces);               // HAND == 2: the pair's activation row, cols bf16
  const int cpe = (a.rows + CR - 1) / CR;                         // chunks per expert
  const int n_chunks = (a.work ? a.n_slots : 1) * cpe;
  const int row_lane = rset * RI * 2 + h;                         // row of this lane in tile 0, i = 0
  const uint32_t w_off = (uint32_t)row_lane * (uint32_t)row_words + (uint32_t)(s * 32 + l) * 4;
  const int sc_off = row_lane * groups + s * 32 + l;
  uint32_t magic;
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));

  struct Work { int e, p_begin, p_end, first_pair, c0, c_first; };
  auto load_work = [&](int chunk) {
    Work w;
    const int ai = chunk / cpe;
    const int4 wk = a.work ? a.work[ai] : make_int4(0, 0, a.n_pairs, 0);
    w.e = __builtin_amdgcn_readfirstlane(wk.x);
    w.p_begin = __builtin_amdgcn_readfirstlane(wk.y);
    w.p_end = __builtin_amdgcn_readfirstlane(wk.z);
    w.first_pair = __builtin_amdgcn_readfirstlane(wk.w);
    w.c_first = (chunk - ai * cpe) * CR;
    w.c0 = w.c_first + CR <= a.rows ? w.c_first : a.rows - CR;  // host guarantees rows >= CR
    return w;
  };
  // group scales of a chunk: CR*groups contiguous bf16 per matrix, copied piece i -> piece i of the buffer
  auto copy_scales = [&](const Work &w, uint4 *dst) {
    const int nwaves = blockDim.x >> 6;
    for (int m = 0; m < MATS; ++m) {
      const uint4 *sg = (const uint4 *)((m ? a.scale1 : a.scale0) + (size_t)w.e * a.expert_scales + (size_t)w.c0 * groups);
      for (int i0 = wave * 64; i0 < n16; i0 += nwaves * 64)
        if (i0 + lane < n16)
          __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)(sg + i0 + lane),
                                           (void __attribute__((address_space(3))) *)(dst + m * n16 + i0), 16, 0, 0);
    }
  };
  auto tile_ptr = [&](const Work &w, int m) {
    return (m ? a.packed1 : a.packed0) + (size_t)w.e * a.expert_words + (size_t)w.c0 * row_words;
  };
  auto load_tile = [&](uint4 (&buf)[MATS][RI], const Work &w, int tile) {
#pragma unroll
    for (int i = 0; i < RI; ++i)
#pragma unroll
      for (int m = 0; m < MATS; ++m)
        buf[m][i] = ld_stream(tile_ptr(w, m) + (size_t)((tile * RT + i * 2) * row_words) + w_off);
  };
  auto load_xraw = [&](uint4 (&xraw)[TT][4], const Work &w, int pc) {
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      const int pi = min(pc + t, w.p_end - 1);
      const int pair = !a.work ? pi : (pi == w.p_begin ? w.first_pair : a.pairs[pi]);
      const uint4 *xp = (const uint4 *)(a.x + (size_t)(pair / a.x_div) * a.cols) + (s * 32 + l) * 4;
#pragma unroll
      for (int q = 0; q < 4; ++q) xraw[t][q] = xp[q];
    }
  };

  // the work of the first chunk at or after c (stride nblocks) whose expert this launch processes; e < 0: none
  auto next_work = [&](int &c) {
    Work w = load_work(c < n_chunks ? c : 0);
    if (c >= n_chunks) w.e = -1;
    if (FILTER) {
      while (w.e >= 0 && (w.p_end - w.p_begin < a.cnt_lo || w.p_end - w.p_begin > a.cnt_hi)) {
        c += nblocks;
        if (c >= n_chunks) { w.e = -1; break; }
        w = load_work(c);
      }
    }
    return w;  // records with work come first: e < 0 ends the list
  };
  int chunk = bid;
  if (chunk >= n_chunks) return;
  Work cur = next_work(chunk);
  if (cur.e < 0) return;
  uint4 bufA[MATS][RI], bufB[MATS][RI];
  uint4 xraw[TT][4];
  int sb = 0;
  copy_scales(cur, sc_base);
  if (active) load_tile(bufA, cur, 0);
  if (HAND == 2) {
    // behind the first tile's requests: a wave's loads return in order, so the answer comes when those have landed
    const uint32_t *src = a.hand + (size_t)cur.first_pair * a.cols + threadIdx.x * 4;
    kxh::hand4 v;
    int polls = 0;
    while (true) {
      kxh::hand_request4(src, v);
      kxh::hand_wait(v);
      if (kxh::hand_tagged(v, a.tag) || kxh::hand_give_up(polls, a.err)) break;
    }
    ((uint2 *)s_xh)[threadIdx.x] = kxh::hand_pack(v);
  } else if (active) {
    load_xraw(xraw, cur, cur.p_begin);
  }
  bool fresh = true;  // the scales of `cur` have not been made visible to the workgroup yet

  while (true) {
    int nchunk = chunk + nblocks;
    bool more = nchunk < n_chunks;
    Work nxt = cur;
    if (more) {
      nxt = next_work(nchunk);
      more = nxt.e >= 0;
    }
    // the other scale buffer was last read in the chunk before this one; every wave is past that chunk's barriers
    if (more) copy_scales(nxt, sc_base + (sb ^ 1) * sc_pieces);
    const uint16_t *sc_lane = (const uint16_t *)(sc_base + sb * sc_pieces) + sc_off;

    for (int pc = cur.p_begin; pc < cur.p_end; pc += TT) {
      XGroup xg[TT];
      if (HAND != 2) {
#pragma unroll
        for (int t = 0; t < TT; ++t) prep_xgroup(xg[t], xraw[t]);
      }
      if (fresh) {  // first chunk of the workgroup: wait for the scale copies of every wave
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        fresh = false;
      }
      if (HAND == 2) {  // the row every thread has collected a piece of
#pragma unroll
        for (int q = 0; q < 4; ++q) xraw[0][q] = ((const uint4 *)s_xh)[(s * 32 + l) * 4 + q];
        prep_xgroup(xg[0], xraw[0]);
      }

      auto compute_tile = [&](uint4 (&buf)[MATS][RI], int tile) {
        float v[NV];
#pragma unroll
        for (int i = 0; i < RI; ++i)
#pragma unroll
          for (int m = 0; m < MATS; ++m) {
            I4Dec dec;
            decode_words(dec, buf[m][i], magic);
            const float sc = kx_bf16_f32(sc_lane[(m * CR + tile * RT + i * 2) * groups]);
#pragma unroll
            for (int t = 0; t < TT; ++t) v[(i * MATS + m) * TT + t] = sc * group_dot(dec, xg[t]);
          }
        kxw::reduce<NV, 32>(v, lane);
        if (kxw::reduce_writer<NV, 32>(lane)) {
#pragma unroll
          for (int j = 0; j < NOUT; ++j) {
            const int idx = kxw::reduce_index<NV, 32>(lane, j);  // (i*MATS + m)*TT + t
            const int t = idx % TT, m = (idx / TT) % MATS, i = idx / (TT * MATS);
            const int rc = tile * RT + row_lane + i * 2;
            part[((m * CR + rc) * TT + t) * ks + s] = v[j];
          }
        }
      };

      if (active)
        for (int tile = 0; tile < nt; tile += 2) {
          if (tile + 1 < nt) load_tile(bufB, cur, tile + 1);
          compute_tile(bufA, tile);
          if (tile + 2 < nt) load_tile(bufA, cur, tile + 2);
          if (tile + 1 < nt) compute_tile(bufB, tile + 1);
        }
      // every load of this wave has landed, the scale copies for the next chunk included; its first tile
      // and activations are requested now and arrive during the epilogue
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      const bool last_pass = pc + TT >= cur.p_end;
      if (HAND == 0 && (!last_pass || more)) {  // a further pass over this chunk (an expert with more than TT pairs), or the next chunk
        const Work &t = last_pass ? nxt : cur;
        load_tile(bufA, t, 0);
        load_xraw(xraw, t, last_pass ? nxt.p_begin : pc + TT);
      } else {  // nothing follows: end the registers' live ranges here
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
          for (int q = 0; q < 4; ++q) xraw[t][q] = make_uint4(0, 0, 0, 0);
        idle();
      }
      __syncthreads();
      // sequential sum over the slices, rounding and epilogue
      for (int idx = threadIdx.x; idx < CR * TT; idx += blockDim.x) {
        const int rc = idx % CR, t = idx / CR;
        if (pc + t < cur.p_end && cur.c0 + rc >= cur.c_first) {  // a moved-back chunk skips the rows it shares
          // the first pair of the group is in the work record: no load in the tail of a one-pair group
          const int pair = !a.work ? pc + t : (pc + t == cur.p_begin ? cur.first_pair : a.pairs[pc + t]);
          const float *p0 = part + ((0 * CR + rc) * TT + t) * ks;
          float y0 = p0[0];
          for (int q = 1; q < ks; ++q) y0 += p0[q];
          float res = y0;
          if (DUAL) {
            const float *p1 = part + ((1 * CR + rc) * TT + t) * ks;
            float y1 = p1[0];
            for (int q = 1; q < ks; ++q) y1 += p1[q];
            res = kx_swiglu(kx_bfround(y0), kx_bfround(y1));
          }
          if (!DUAL && a.tail.counter)  // read back by another workgroup of this launch
            kx_arrive_store(a.out + (size_t)pair * a.rows + cur.c0 + rc, kx_bf16_rne(res));
          else
            a.out[(size_t)pair * a.rows + cur.c0 + rc] = kx_bf16_rne(res);
          if (HAND == 1) kxh::hand_store(a.hand + (size_t)pair * a.rows + cur.c0 + rc, a.tag, kx_bf16_rne(res));
        }
      }
      __syncthreads();  // `part` is free again; the next chunk's scale copies are visible to every wave
    }
    if (!more || HAND != 0) break;
    cur = nxt;
    chunk = nchunk;
    sb ^= 1;
  }
}

template <bool DUAL, int TT, int KS_T, int MAXT, int WPE, bool FILTER, int CM = 1>
__global__ void __launch_bounds__(MAXT) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) i4_gemv_k(I4Args a) {
  extern __shared__ float lds[];
  i4_body<DUAL, TT, KS_T, FILTER, CM>(a, blockIdx.x, gridDim.x, lds, [] {});
}

// The routed down GEMV of one token and the shared expert's down GEMV ([rows, 2048] bf16) in one launch.  Workgroup b
// takes routed chunk b (112 rows of one expert) and then chunk b of the shared matrix (16 rows), whose weights and
// first tile and activations it requests where the routed chunk's last loads have landed, so that they arrive during
// its epilogue.
// Both chunks finish through moe_tail_arrive: the launch leaves the layer's output in x.
// The shared chunk is computed as kx_gemv_launch computes it for this shape (4 slice waves x 2 row sets, 4 rows per
// wave and tile, 2 tiles): lane partials over 8 columns, butterfly over the wave, slices summed left to right.
template <int HAND>
__device__ __forceinline__ void down_shared_body(const I4Args &a, const KxGemvArgs &g, int n_i4, int n_g, float *lds) {
  constexpr int S = 4, RI = 4, RT = 8, CR = 16;  // two tiles of RT rows per chunk
  const int bid = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wslot = wave & 3, rset = wave >> 2;
  const bool has_g = bid < n_g;
  const uint32_t col = (uint32_t)wslot * 512u + (uint32_t)lane * 8u;
  uint4 gw0[RI], gx = make_uint4(0, 0, 0, 0);
  bool loaded = false;
  auto load_tile = [&](uint4 (&w)[RI], int t) {
#pragma unroll
    for (int i = 0; i < RI; ++i) w[i] = kxg::ld_stream16(g.w0 + (size_t)(bid * CR + t * RT + rset * RI + i) * g.cols + col);
  };
  auto load_shared = [&]() {  // first tile and the activations
    if (has_g && !loaded) {
      load_tile(gw0, 0);
      gx = *(const uint4 *)(g.x + col);
    }
    loaded = true;
  };
  // one routed chunk per workgroup (the host launches one workgroup per chunk): its row block, if it has work
  constexpr int BLOCK = i4_chunk_rows(false, 16);
  int routed_blk = -1;
  if (bid < n_i4) {
    i4_body<false, 1, 2, false, 1, HAND>(a, bid, n_i4, lds, load_shared);
    if (a.work[bid / (a.rows / BLOCK)].x >= 0) routed_blk = bid % (a.rows / BLOCK);
  }
  load_shared();  // a workgroup without routed work
  if (!has_g) {
    if (routed_blk >= 0) moe_tail_arrive(a.tail, routed_blk, -1, BLOCK, a.rows, a.out);
    return;
  }
  uint4 gw1[RI];
  load_tile(gw1, 1);
  float xs[8];
  kxg::unpack8(xs, gx);
  auto compute_tile = [&](const uint4 (&w)[RI], int t) {
    float v[RI];
#pragma unroll
    for (int i = 0; i < RI; ++i) {
      float wf[8];
      kxg::unpack8(wf, w[i]);
      float acc = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(wf[e], xs[e], acc);
      v[i] = acc;
    }
    kxw::reduce<RI, 64>(v, lane);
    if (kxw::reduce_writer<RI, 64>(lane)) {
#pragma unroll
      for (int j = 0; j < kxw::reduce_out<RI, 64>(); ++j) {
        const int i = kxw::reduce_index<RI, 64>(lane, j);
        lds[(t * RT + rset * RI + i) * S + wslot] = v[j];
      }
    }
  };
  compute_tile(gw0, 0);
  compute_tile(gw1, 1);
  __syncthreads();
  if (threadIdx.x < CR) {
    const float *p = lds + threadIdx.x * S;
    float y = p[0];
    for (int q = 1; q < S; ++q) y += p[q];
    kx_arrive_store((uint16_t *)g.out + bid * CR + threadIdx.x, kx_bf16_rne(y));
  }
  moe_tail_arrive(a.tail, routed_blk, bid * CR / BLOCK, BLOCK, a.rows, a.out);
}

__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) i4_down_shared_k(I4Args a, KxGemvArgs g, int n_i4,
                                                                                                 int n_g) {
  extern __shared__ float lds[];
  down_shared_body<0>(a, g, n_i4, n_g, lds);
}

// The routed experts of one token as one launch: workgroup b computes chunk b of gate/up (32 rows of both matrices
// of one expert, SwiGLU) with seven of its eight waves, hands the 32 values over as tagged words, and goes on as
// workgroup b of the launch above with the activations of its down chunk -- the expert's 2048 mid values, from the 64
// workgroups of the same expert -- collected from those words.  As launches of their own the second one cannot ask
// for a byte before the first has drained; here a workgroup requests its down chunk's scales and first tile, then
// polls.  Every workgroup must be resident (two per CU): the launcher checks CUs, LDS and the grid.
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) i4_routed_shared_k(I4Args gu, I4Args a, KxGemvArgs g,
                                                                                                   int n_i4, int n_g) {
  extern __shared__ float lds[];
  i4_body<true, 1, 7, false, 1, 1>(gu, blockIdx.x, gridDim.x, lds, [] {});
  __syncthreads();  // a workgroup without a gate/up chunk returns from the body early; the LDS changes hands here
  down_shared_body<2>(a, g, n_i4, n_g, lds);
}

struct I4Launch {
  int ks, rs, nt, threads, cr;
  size_t lds;
};

// one_chunk: every workgroup has one chunk (the grid is the chunk list), so the second scale buffer, which holds the
// next chunk's scales, is left out
int plan(int cols, int rows, int mats, int tt, I4Launch &pl, int chunk_mult = 1, bool one_chunk = false) {
  KX_REQUIRE(cols > 0 && cols % 1024 == 0, "kx_i4: cols=%d must be a positive multiple of 1024", cols);
  KX_REQUIRE(rows >= 4, "kx_i4: rows=%d must be at least 4", rows);
  pl.ks = cols / 1024;
  KX_REQUIRE(pl.ks <= 16, "kx_i4: cols=%d exceeds 16384", cols);
  pl.rs = pl.ks >= 5 ? 1 : (8 / pl.ks);
  while (pl.rs > 1 && pl.rs * 4 > rows) pl.rs >>= 1;  // a tile must fit in the matrix
  pl.threads = pl.ks * pl.rs * 64;
  const int rt = pl.rs * 2 * I4_RI;
  // chunk: 32 rows of both matrices (gate/up) or 64 rows of one
  int nt = i4_chunk_rows(mats == 2, rt) / rt;
  nt = nt < 1 ? 1 : nt;
  if (chunk_mult > 1 && rows % (rt * nt * chunk_mult) == 0) nt *= chunk_mult;
  while (nt > 1 && rt * nt > rows) --nt;
  pl.nt = nt;
  pl.cr = rt * nt;
  const size_t sc_pieces = ((size_t)mats * pl.cr * (cols / 32) / 8 + 63) & ~(size_t)63;  // 16-byte pieces per scale buffer
  pl.lds = (((size_t)mats * pl.cr * tt * pl.ks + 3) & ~(size_t)3) * sizeof(float) + (one_chunk ? 1 : 2) * sc_pieces * 16;
  KX_REQUIRE(pl.lds <= 160 * 1024, "kx_i4: cols=%d needs %zu bytes of LDS", cols, pl.lds);
  return KX_OK;
}

template <bool DUAL, int KS_T, int MAXT>
void launch_tt(const I4Args &a, int tt, dim3 g, dim3 b, size_t lds, hipStream_t st) {
  // waves per SIMD the register budget is held to: two 7- or 8-wave workgroups per CU
  // for one or two tokens per pass, fewer when four tokens' activations live in registers
  const bool filter = a.cnt_lo > 0 || a.cnt_hi != 0x7fffffff;
  if (tt == 1) {
    if (filter) hipLaunchKernelGGL((i4_gemv_k<DUAL, 1, KS_T, MAXT, 4, true>), g, b, lds, st, a);
    else hipLaunchKernelGGL((i4_gemv_k<DUAL, 1, KS_T, MAXT, 4, false>), g, b, lds, st, a);
  } else if (tt == 2) {
    hipLaunchKernelGGL((i4_gemv_k<DUAL, 2, KS_T, MAXT, 4, true>), g, b, lds, st, a);
  } else {
    hipLaunchKernelGGL((i4_gemv_k<DUAL, 4, KS_T, MAXT, (MAXT > 512 ? 4 : 2), true>), g, b, lds, st, a);
  }
}

}  // namespace

// Launches the fused gate/up (dual) or single-matrix GEMV over a bucketed pair list.
// tt: tokens per pass (1, 2 or 4).  n_slots: records in `work`.
int kx_i4_launch(bool dual, const uint32_t *packed0, const uint16_t *scale0, const uint32_t *packed1,
                 const uint16_t *scale1, const uint16_t *x, uint16_t *out, const int4 *work,
                 const int *pairs, int n_pairs, int rows, int cols, int x_div, size_t expert_words,
                 size_t expert_scales, int tt, int n_slots, int cnt_lo, int cnt_hi, hipStream_t st, int chunk_mult) {
  I4Launch pl;
  // chunks of twice the rows: for the one-matrix kernel over many work records, where a 112-row chunk (114 KB at
  // K = 2048) is over before the workgroup's start-up is paid for (routed down at 32 tokens: 0.367 -> 0.33 ms)
  const bool filter = cnt_lo > 0 || cnt_hi != 0x7fffffff;
  int cm = (chunk_mult == 2 && !dual && work && tt <= 2 && cols == 2048) ? 2 : 1;
  // the gate/up kernel over a per-pair list: 64-row chunks (458 KB) with one scale buffer, when the grid holds them all
  const bool dual2 = chunk_mult == 2 && dual && work && tt == 1 && !filter && cols == 7168 && rows % 64 == 0 &&
                     (long)n_slots * (rows / 64) <= 32768;
  if (dual2) cm = 2;
  int rc = plan(cols, rows, dual ? 2 : 1, tt, pl, cm, dual2);
  if (rc) return rc;
  I4Args a = {};
  a.packed0 = packed0; a.scale0 = scale0; a.packed1 = packed1; a.scale1 = scale1;
  a.x = x; a.out = out; a.work = work; a.pairs = pairs; a.n_pairs = n_pairs; a.n_slots = n_slots;
  a.rows = rows; a.cols = cols; a.x_div = x_div; a.ks = pl.ks; a.rs = pl.rs; a.nt = pl.nt;
  a.expert_words = expert_words; a.expert_scales = expert_scales;
  a.cnt_lo = cnt_lo; a.cnt_hi = cnt_hi;
  a.tail = KxMoeTail{};
  long chunks = (long)n_slots * kx_cdiv(rows, pl.cr);
  dim3 g((unsigned)(chunks < 32768 ? chunks : 32768)), b(pl.threads);
  const bool full = pl.rs == (pl.ks >= 5 ? 1 : 8 / pl.ks) && pl.nt == i4_chunk_rows(dual, pl.rs * 4) / (pl.rs * 4);
  const bool full2 = cm == 2 && pl.ks == 2 && pl.rs == 4 && pl.nt == 2 * (i4_chunk_rows(false, 16) / 16);
  if (dual2 && pl.ks == 7 && pl.rs == 1 && pl.nt == 16) {
    hipLaunchKernelGGL((i4_gemv_k<true, 1, 7, 448, 4, false, 2>), g, b, pl.lds, st, a);
  } else if (full2) {              // Kimi-K2 down over many records: 224-row chunks
    if (tt == 2) hipLaunchKernelGGL((i4_gemv_k<false, 2, 2, 512, 4, true, 2>), g, b, pl.lds, st, a);
    else if (filter) hipLaunchKernelGGL((i4_gemv_k<false, 1, 2, 512, 4, true, 2>), g, b, pl.lds, st, a);
    else hipLaunchKernelGGL((i4_gemv_k<false, 1, 2, 512, 4, false, 2>), g, b, pl.lds, st, a);
  } else if (full && pl.ks == 7) {        // Kimi-K2 gate/up: K = 7168
    if (dual) launch_tt<true, 7, 448>(a, tt, g, b, pl.lds, st);
    else launch_tt<false, 7, 448>(a, tt, g, b, pl.lds, st);
  } else if (full && pl.ks == 2) {  // Kimi-K2 down: K = 2048
    if (dual) launch_tt<true, 2, 512>(a, tt, g, b, pl.lds, st);
    else launch_tt<false, 2, 512>(a, tt, g, b, pl.lds, st);
  } else if (pl.threads <= 512) {
    if (dual) launch_tt<true, 0, 512>(a, tt, g, b, pl.lds, st);
    else launch_tt<false, 0, 512>(a, tt, g, b, pl.lds, st);
  } else {
    if (dual) launch_tt<true, 0, 1024>(a, tt, g, b, pl.lds, st);
    else launch_tt<false, 0, 1024>(a, tt, g, b, pl.lds, st);
  }
  KX_LAUNCH_CHECK();
  return KX_OK;
}

int kx_i4_down_shared_launch(const uint32_t *packed, const uint16_t *scale, const uint16_t *x, uint16_t *out, const int4 *work,
                             const int *pairs, int rows, int cols, int x_div, size_t expert_words, size_t expert_scales,
                             int n_slots, KxGemvArgs shared, KxMoeTail tail, bool *fused, hipStream_t st) {
  *fused = false;
  if (tail.tokens != 1 || shared.tokens != 1 || !tail.counter || !work || shared.rows != rows) return KX_OK;
  I4Launch pl;
  int rc = plan(cols, rows, 1, 1, pl);
  if (rc) return rc;
  if (!(pl.ks == 2 && pl.rs == 4 && pl.cr == i4_chunk_rows(false, 16) && rows % pl.cr == 0)) return KX_OK;
  // the kernel computes the shared chunk with the launch shape kx_gemv_launch gives this matrix
  int ri;
  shared.out = (void *)tail.sy;
  shared.out_stride = rows;
  if (kx_gemv_plan(KX_EPI_BF16, shared, &ri) < 0) return KX_ERR_ARG;
  if (!(shared.cols == 2048 && ri == 4 && shared.nw == 4 && shared.rs == 2) || shared.row_block || shared.norm_w) return KX_OK;
  const int g_cr = 16;
  if (pl.cr % g_cr || rows % g_cr) return KX_OK;
  tail.shared_chunks = pl.cr / g_cr;
  const long n_i4 = (long)n_slots * (rows / pl.cr), n_g = rows / g_cr;
  if (n_i4 > 32768 || n_g > 32768) return KX_OK;
  const size_t lds_g = (size_t)g_cr * 4 * sizeof(float);
  const size_t lds = pl.lds > lds_g ? pl.lds : lds_g;
  I4Args a = {};
  a.packed0 = packed; a.scale0 = scale; a.packed1 = nullptr; a.scale1 = nullptr;
  a.x = x; a.out = out; a.work = work; a.pairs = pairs; a.n_pairs = 0; a.n_slots = n_slots;
  a.rows = rows; a.cols = cols; a.x_div = x_div; a.ks = pl.ks; a.rs = pl.rs; a.nt = pl.nt;
  a.expert_words = expert_words; a.expert_scales = expert_scales;
  a.cnt_lo = 0; a.cnt_hi = 0x7fffffff;
  a.tail = tail;
  hipLaunchKernelGGL(i4_down_shared_k, dim3((unsigned)(n_i4 > n_g ? n_i4 : n_g)), dim3(512), lds, st, a, shared, (int)n_i4, (int)n_g);
  KX_LAUNCH_CHECK();
  *fused = true;
  return KX_OK;
}

// The routed experts of one token -- gate/up + SwiGLU, down, the shared expert's down GEMV, combine, residual -- as one
// launch (i4_routed_shared_k).  x: the normed row [hidden]; mid: [n_slots, inter] (also written, as the separate
// launches leave it); hand: n_slots * inter words; tag in [1, 65535], different from the previous launch's on `hand`;
// err: the flag a workgroup sets when it gives a wait up.  *fused = false and nothing launched when the shapes or the
// device do not allow the resident form.
int kx_i4_routed_shared_launch(const uint32_t *gate_packed, const uint16_t *gate_scale, const uint32_t *up_packed, const uint16_t *up_scale,
                               const uint32_t *down_packed, const uint16_t *down_scale, const uint16_t *x, uint16_t *mid, uint16_t *eout,
                               const int4 *work, const int *pairs, int hidden, int inter, int topk, int n_slots, KxGemvArgs shared,
                               KxMoeTail tail, uint32_t *hand, uint32_t tag, int *err, bool *fused, hipStream_t st) {
  *fused = false;
  if (tail.tokens != 1 || shared.tokens != 1 || !tail.counter || !work || shared.rows != hidden || !hand || !err || tag < 1 || tag > 65535)
    return KX_OK;
  const int cus = kx_device_cus();  // 0 (query failed): the resident form is declined below
  I4Launch pu, pd;
  int rc = plan(hidden, inter, 2, 1, pu);
  if (rc) return rc;
  if ((rc = plan(inter, hidden, 1, 1, pd))) return rc;
  // gate/up: 7 slice waves, chunks of 32 rows; down: 2 slices x 4 row sets, chunks of 112 rows, 4 * 512 columns
  if (!(pu.ks == 7 && pu.rs == 1 && pu.cr == 32 && inter % pu.cr == 0)) return KX_OK;
  if (!(pd.ks == 2 && pd.rs == 4 && pd.cr == i4_chunk_rows(false, 16) && hidden % pd.cr == 0 && inter == 4 * 512)) return KX_OK;
  int ri;
  shared.out = (void *)tail.sy;
  shared.out_stride = hidden;
  if (kx_gemv_plan(KX_EPI_BF16, shared, &ri) < 0) return KX_ERR_ARG;
  if (!(shared.cols == 2048 && ri == 4 && shared.nw == 4 && shared.rs == 2) || shared.row_block || shared.norm_w) return KX_OK;
  const int g_cr = 16;
  if (pd.cr % g_cr || hidden % g_cr) return KX_OK;
  tail.shared_chunks = pd.cr / g_cr;
  const long n_gu = (long)n_slots * (inter / pu.cr), n_i4 = (long)n_slots * (hidden / pd.cr), n_g = hidden / g_cr;
  // every workgroup waits for others of the launch: all of them resident, two per CU
  const size_t lds_d = pd.lds + (size_t)inter * 2, lds_g = (size_t)g_cr * 4 * sizeof(float);
  size_t lds = pu.lds > lds_d ? pu.lds : lds_d;
  lds = lds > lds_g ? lds : lds_g;
  if (n_gu != n_i4 || n_g > n_i4 || n_i4 > 2L * cus || lds > 78 * 1024) return KX_OK;
  static bool attr_set = false;
  if (!attr_set) {
    KX_HIP(hipFuncSetAttribute((const void *)i4_routed_shared_k, hipFuncAttributeMaxDynamicSharedMemorySize, 78 * 1024));
    attr_set = true;
  }
  I4Args u = {};
  u.packed0 = gate_packed; u.scale0 = gate_scale; u.packed1 = up_packed; u.scale1 = up_scale;
  u.x = x; u.out = mid; u.work = work; u.pairs = pairs; u.n_pairs = 0; u.n_slots = n_slots;
  u.rows = inter; u.cols = hidden; u.x_div = topk; u.ks = pu.ks; u.rs = pu.rs; u.nt = pu.nt;
  u.expert_words = (size_t)inter * (hidden / 8); u.expert_scales = (size_t)inter * (hidden / 32);
  u.cnt_lo = 0; u.cnt_hi = 0x7fffffff;
  u.tail = KxMoeTail{};
  u.hand = hand; u.tag = tag; u.err = err;
  I4Args d = {};
  d.packed0 = down_packed; d.scale0 = down_scale;
  d.x = mid; d.out = eout; d.work = work; d.pairs = pairs; d.n_pairs = 0; d.n_slots = n_slots;
  d.rows = hidden; d.cols = inter; d.x_div = 1; d.ks = pd.ks; d.rs = pd.rs; d.nt = pd.nt;
  d.expert_words = (size_t)hidden * (inter / 8); d.expert_scales = (size_t)hidden * (inter / 32);
  d.cnt_lo = 0; d.cnt_hi = 0x7fffffff;
  d.tail = tail;
  d.hand = hand; d.tag = tag; d.err = err;
  hipLaunchKernelGGL(i4_routed_shared_k, dim3((unsigned)n_i4), dim3(512), lds, st, u, d, shared, (int)n_i4, (int)n_g);
  KX_LAUNCH_CHECK();
  *fused = true;
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
  return kx_i4_launch(false, (const uint32_t *)d_packed, (const uint16_t *)d_scale, nullptr, nullptr,
                      (const uint16_t *)d_x, (uint16_t *)d_y, nullptr, nullptr, tokens, rows, cols, 1, 0, 0, tt, 1, 0, 0x7fffffff,
                      kx_stream(stream));
}
