// kx_gemv_body.h -- the bf16-weight GEMV as a device function: one workgroup's share of the work.
// Used by the GEMV kernels of kx_dense.hip: the plain one, the pair that runs the shared expert's gate/up and the
// router in one launch, and the q_b GEMV that finishes the query (W_UK absorb, RoPE) in the same launch.
#pragma once
#include "kx_arrive.h"
#include "kx_common.h"
#include "kx_dense.h"
#include "kx_math.h"
#include "kx_wave.h"

namespace kxg {

typedef unsigned int kx_u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint4 ld_stream16(const uint16_t *p) {
  kx_u32x4 v = __builtin_nontemporal_load((const kx_u32x4 *)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float bf_lo(uint32_t u) { return kx_bits_f32(u << 16); }
__device__ __forceinline__ float bf_hi(uint32_t u) { return kx_bits_f32(u & 0xffff0000u); }

__device__ __forceinline__ void unpack8(float (&f)[8], uint4 u) {
  f[0] = bf_lo(u.x); f[1] = bf_hi(u.x); f[2] = bf_lo(u.y); f[3] = bf_hi(u.y);
  f[4] = bf_lo(u.z); f[5] = bf_hi(u.z); f[6] = bf_lo(u.w); f[7] = bf_hi(u.w);
}

// ---- GEMV -------------------------------------------------------------------------
// A workgroup of nw*rs waves takes chunks of nt tiles of RT = rs*RI rows.  Wave
// (wslot, rset) owns the 512-column slices wslot, wslot+nw, ... of rows rset*RI ..
// rset*RI+RI-1 of each tile, one slice per pass over the chunk.  The 16-byte weight
// loads of tile i+1 are in flight while tile i is computed; partial sums per (row,
// token, slice) go to LDS and are summed left to right over the slices at the end of
// the chunk, where the epilogue runs.  A last chunk that would run past the matrix is
// moved back to end at the last row; the rows it shares with the previous chunk are
// computed twice but written once, by the previous chunk.
template <int MATS, int RI, int TT>
__device__ __forceinline__ void gemv_body(const KxGemvArgs &a, const int bid, const int nblocks,
                                          float *part /* LDS [mats][CR][tokens][S] */) {
  constexpr int NV = RI * MATS * TT;
  constexpr int NOUT = kxw::reduce_out<NV, 64>();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int S = a.cols >> 9, T = a.tokens;
  const int wslot = wave % a.nw, rset = wave / a.nw;
  const int RT = a.rs * RI, CR = RT * a.nt;
  const int n_chunks = (a.rows + CR - 1) / CR;
  const bool x_once = T <= TT;  // activations stay in registers for the whole chunk
  const uint16_t *wm[2] = {a.w0, MATS == 2 ? a.w1 : a.w0};

  // (chunk, slice) -> first row of the chunk, its row block, this lane's column, this wave's weight rows
  struct Item { int c0, blk; uint32_t col; const uint16_t *wb[2]; };
  auto item = [&](int chunk, int s) {
    Item it;
    it.c0 = chunk * CR;
    it.c0 = it.c0 + CR <= a.rows ? it.c0 : a.rows - CR;  // host guarantees rows >= CR
    it.col = (uint32_t)s * 512u + (uint32_t)lane * 8u;
    it.blk = a.row_block ? it.c0 / a.row_block : 0;
    const int wrow0 = a.row_block ? it.blk * a.w_block_stride + a.w_block_off + (it.c0 - it.blk * a.row_block) : it.c0;
    it.wb[0] = wm[0] + (size_t)(wrow0 + rset * RI) * a.cols;
    it.wb[1] = wm[1] + (size_t)(wrow0 + rset * RI) * a.cols;
    return it;
  };
  auto load_tile = [&](uint4 (&buf)[MATS][RI], const Item &it, int tile) {
#pragma unroll
    for (int i = 0; i < RI; ++i)
#pragma unroll
      for (int m = 0; m < MATS; ++m)
        buf[m][i] = ld_stream16(it.wb[m] + (size_t)((tile * RT + i) * a.cols) + it.col);
  };
  // The work of a wave is one sequence of steps (chunk, slice, tile), tiles innermost, in which the
  // loads of step i+1 (weights, and the raw activations when it starts a slice) are in flight while
  // step i is computed; the first step's loads are requested before the prologue.
  struct Pos { int chunk, s, tile; };
  auto advance = [&](Pos p) {
    if (++p.tile == a.nt) {
      p.tile = 0;
      p.s += a.nw;
      if (p.s >= S) { p.s = wslot; p.chunk += nblocks; }
    }
    return p;
  };
  struct XRaw { uint4 x[TT]; uint4 g; };
  // activations of a slice are fetched one step ahead (not in the variant whose registers are full)
  const bool x_pref = x_once && !a.mla_po && !(MATS == 2 && RI == 2);
  auto load_xraw = [&](XRaw &r, const Item &it) {
    const uint16_t *xb = a.x + (size_t)it.blk * a.x_block_stride;
#pragma unroll
    for (int t = 0; t < TT; ++t) r.x[t] = *(const uint4 *)(xb + (size_t)min(t, T - 1) * a.x_stride + it.col);
    if (a.norm_w) r.g = *(const uint4 *)(a.norm_w + it.col);
  };
  uint4 bufA[MATS][RI], bufB[MATS][RI];
  XRaw xrA, xrB;
  Pos cur = {bid, wslot, 0};
  if (cur.chunk >= n_chunks) return;  // whole workgroups only: the host launches at most n_chunks of them
  Item itc = item(cur.chunk, cur.s);
  load_tile(bufA, itc, 0);
  if (x_pref) load_xraw(xrA, itc);

  // Optional prologue: RMSNorm of the activation rows (rmsnorm_k's schedule: 256 threads own the
  // 8-element chunks t, t+256, ...; butterfly per wave; ((w0+w1)+w2)+w3).  Every workgroup
  // computes the row scales; the normalised values are formed when the activations are loaded.
  __shared__ float n_ws[4];
  __shared__ float n_scale[4];
  if (a.norm_w) {
    const int chunks = a.cols >> 3;
    for (int t = 0; t < T; ++t) {
      const uint16_t *xr = a.x + (size_t)t * a.x_stride;
      float v = 0.0f;
      if (threadIdx.x < 256)
        for (int c = threadIdx.x; c < chunks; c += 256) {
          float f[8];
          unpack8(f, ((const uint4 *)xr)[c]);
#pragma unroll
          for (int e = 0; e < 8; ++e) v = __builtin_fmaf(f[e], f[e], v);
        }
      float vv[1] = {v};
      kxw::reduce<1, 64>(vv, lane);
      if (lane == 0 && wave < 4) n_ws[wave] = vv[0];
      __syncthreads();
      if (threadIdx.x == 0) n_scale[t] = kx_rsqrtf((((n_ws[0] + n_ws[1]) + n_ws[2]) + n_ws[3]) / (float)a.cols + a.norm_eps);
      __syncthreads();
    }
    if (a.norm_out && bid == 0)  // one workgroup also stores the normalised rows for later kernels
      for (int t = 0; t < T; ++t) {
        const uint16_t *xr = a.x + (size_t)t * a.x_stride;
        uint16_t *yr = a.norm_out + (size_t)t * a.cols;
        const float sc = n_scale[t];
        for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
          float f[8], g[8];
          unpack8(f, ((const uint4 *)xr)[c]);
          unpack8(g, ((const uint4 *)a.norm_w)[c]);
          uint32_t o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o[e] = (uint32_t)kx_bf16_rne(kx_bfround(f[2 * e] * sc) * g[2 * e]) |
                   ((uint32_t)kx_bf16_rne(kx_bfround(f[2 * e + 1] * sc) * g[2 * e + 1]) << 16);
          ((uint4 *)yr)[c] = make_uint4(o[0], o[1], o[2], o[3]);
        }
      }
  }

  float xs[TT][8];
  // activations of tokens t0 .. t0+TT-1 for the slice of `it`, straight from memory
  auto load_x = [&](const Item &it, int t0) {
    const uint32_t col = it.col;
    const int blk = it.blk;
    const uint16_t *xb = a.x + (size_t)blk * a.x_block_stride;
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      const int tok = min(t0 + t, T - 1);
      if (a.mla_po) {
            // activations = merged attention partials of head `blk` (mla_combine's arithmetic):
            // M = max M_j; w_j = exp(M_j - M); Z = fma(Z_j, w_j, Z); O = fma(O_j, w_j, O); x = bf(O / Z).
            // Lane j holds span j's (M_j, Z_j, w_j); the O_j rows are fetched four spans at a time.
            const int spans = a.mla_spans;
            const size_t idx0 = (size_t)tok * spans * a.mla_heads + blk;
            const size_t my = idx0 + (size_t)min(lane, spans - 1) * a.mla_heads;
            const float mj = a.mla_pm[my], zj = a.mla_pz[my];
            const float M = kxw::wave_max_f32(lane < spans ? mj : -__builtin_inff());
            const float wj = kx_expf(mj - M);
            float Z = 0.0f, O[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int j = 0; j < spans; ++j)
              Z = __builtin_fmaf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, zj), j)),
                                 __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), j)), Z);
            for (int j0 = 0; j0 < spans; j0 += 4) {
              float4 o0[4], o1[4];
#pragma unroll
              for (int u = 0; u < 4; ++u) {
                const float4 *o = (const float4 *)(a.mla_po + (idx0 + (size_t)min(j0 + u, spans - 1) * a.mla_heads) * a.cols + col);
                o0[u] = o[0];
                o1[u] = o[1];
              }
#pragma unroll
              for (int u = 0; u < 4; ++u) {
                if (j0 + u < spans) {
                  const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), j0 + u));
                  O[0] = __builtin_fmaf(o0[u].x, w, O[0]); O[1] = __builtin_fmaf(o0[u].y, w, O[1]);
                  O[2] = __builtin_fmaf(o0[u].z, w, O[2]); O[3] = __builtin_fmaf(o0[u].w, w, O[3]);
                  O[4] = __builtin_fmaf(o1[u].x, w, O[4]); O[5] = __builtin_fmaf(o1[u].y, w, O[5]);
                  O[6] = __builtin_fmaf(o1[u].z, w, O[6]); O[7] = __builtin_fmaf(o1[u].w, w, O[7]);
                }
              }
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) xs[t][e] = kx_bfround(O[e] / Z);
      } else {
        unpack8(xs[t], *(const uint4 *)(xb + (size_t)tok * a.x_stride + col));
        if (a.norm_w) {
          float g[8];
          unpack8(g, *(const uint4 *)(a.norm_w + col));
          const float sc = n_scale[tok];
#pragma unroll
          for (int e = 0; e < 8; ++e) xs[t][e] = kx_bfround(kx_bfround(xs[t][e] * sc) * g[e]);
        }
      }
    }
  };
  // the same from the prefetched raw values
  auto form_x = [&](const XRaw &r) {
    float g[8];
    if (a.norm_w) unpack8(g, r.g);
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      unpack8(xs[t], r.x[t]);
      if (a.norm_w) {
        const float sc = n_scale[min(t, T - 1)];
#pragma unroll
        for (int e = 0; e < 8; ++e) xs[t][e] = kx_bfround(kx_bfround(xs[t][e] * sc) * g[e]);
      }
    }
  };
  auto compute_tile = [&](uint4 (&buf)[MATS][RI], const Item &it, int s, int tile) {
    for (int t0 = 0; t0 < T; t0 += TT) {
      if (!x_once) load_x(it, t0);
      float v[NV];
#pragma unroll
      for (int i = 0; i < RI; ++i)
#pragma unroll
        for (int m = 0; m < MATS; ++m) {
          float wf[8];
          unpack8(wf, buf[m][i]);
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            float acc = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(wf[e], xs[t][e], acc);
            v[(i * MATS + m) * TT + t] = acc;
          }
        }
      kxw::reduce<NV, 64>(v, lane);
      if (kxw::reduce_writer<NV, 64>(lane)) {
#pragma unroll
        for (int j = 0; j < NOUT; ++j) {
          const int idx = kxw::reduce_index<NV, 64>(lane, j);  // (i*MATS + m)*TT + t
          const int t = idx % TT, m = (idx / TT) % MATS, i = idx / (TT * MATS);
          const int rc = tile * RT + rset * RI + i, tok = t0 + t;
          if (tok < T) part[((m * CR + rc) * T + tok) * S + s] = v[j];
        }
      }
    }
  };
  // end of a chunk: the slices of every (row, token) are summed left to right and the epilogue runs
  auto chunk_end = [&](int chunk, int c0) {
    __syncthreads();
    for (int idx = threadIdx.x; idx < CR * T; idx += blockDim.x) {
      const int rc = idx % CR, tok = idx / CR;
      const int row = c0 + rc;
      if (row < chunk * CR) continue;  // rows of a moved-back last chunk that the previous chunk owns
      // the slice sums are read eight at a time (one wait per eight instead of one per addition) and added in order
      auto slice_sum = [&](const float *p) {
        float y = p[0];
        for (int q0 = 1; q0 < S; q0 += 8) {
          float t[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) t[u] = p[min(q0 + u, S - 1)];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (q0 + u < S) y += t[u];
        }
        return y;
      };
      const float y0 = slice_sum(part + ((0 * CR + rc) * T + tok) * S);
      float y1 = 0.0f;
      if (MATS == 2) y1 = slice_sum(part + ((1 * CR + rc) * T + tok) * S);
      switch (a.epi) {
        case KX_EPI_BF16:
          if (a.flags & KX_GEMV_COHERENT_OUT)
            kx_arrive_store((uint16_t *)a.out + (size_t)tok * a.out_stride + row, kx_bf16_rne(y0));
          else
            ((uint16_t *)a.out)[(size_t)tok * a.out_stride + row] = kx_bf16_rne(y0);
          break;
        case KX_EPI_F32:
          if (a.flags & KX_GEMV_COHERENT_OUT)  // read back by another workgroup of this launch: store through to memory
            kx_arrive_store((float *)a.out + (size_t)tok * a.out_stride + row, y0);
          else
            ((float *)a.out)[(size_t)tok * a.out_stride + row] = y0;
          break;
        case KX_EPI_SWIGLU:
          ((uint16_t *)a.out)[(size_t)tok * a.out_stride + row] = kx_bf16_rne(kx_swiglu(kx_bfround(y0), kx_bfround(y1)));
          break;
        case KX_EPI_RESID: {  // x = bf(x + bf(y))  (add_k, :248-251)
          uint16_t *xr = (uint16_t *)a.out + (size_t)tok * a.out_stride + row;
          *xr = kx_bf16_rne(kx_bf16_f32(*xr) + kx_bfround(y0));
          break;
        }
        case KX_EPI_MOE_COMBINE: {
          // down = bf(sum_slot y_slot * w_slot) in slot order (:868,:871), then
          // down = bf(down + bf(shared)) (:684), then x = bf(x + down) (:877)
          float acc = 0.0f;
          for (int k = 0; k < a.topk; ++k)
            acc = __builtin_fmaf(kx_bf16_f32(a.expert_out[((size_t)tok * a.topk + k) * a.rows + row]),
                                 a.route_w[(size_t)tok * a.topk + k], acc);
          const float down = kx_bfround(kx_bfround(acc) + kx_bfround(y0));
          uint16_t *xr = (uint16_t *)a.out + (size_t)tok * a.out_stride + row;
          *xr = (a.flags & 1u) ? kx_bf16_rne(down) : kx_bf16_rne(kx_bf16_f32(*xr) + down);
          break;
        }
        case KX_EPI_ARGMAX:  // bf16-rounded logits; a second kernel reduces them
          ((float *)a.out)[(size_t)tok * a.out_stride + row] = kx_bfround(y0);
          break;
      }
    }
    __syncthreads();
  };
  auto step = [&](uint4 (&buf)[MATS][RI], const XRaw &xr, const Pos &p, const Item &it, bool last_of_chunk) {
    if (x_once && p.tile == 0) {
      if (x_pref) form_x(xr);
      else load_x(it, 0);
    }
    compute_tile(buf, it, p.s, p.tile);
    if (last_of_chunk) chunk_end(p.chunk, it.c0);
  };
  while (true) {
    Pos nxt = advance(cur);
    bool more = nxt.chunk < n_chunks;
    Item itn = itc;
    if (more) {
      if (nxt.tile == 0) itn = item(nxt.chunk, nxt.s);
      load_tile(bufB, itn, nxt.tile);
      if (x_pref && nxt.tile == 0) load_xraw(xrB, itn);
    }
    step(bufA, xrA, cur, itc, nxt.chunk != cur.chunk);
    if (!more) break;
    cur = nxt;
    itc = itn;
    nxt = advance(cur);
    more = nxt.chunk < n_chunks;
    if (more) {
      if (nxt.tile == 0) itn = item(nxt.chunk, nxt.s);
      load_tile(bufA, itn, nxt.tile);
      if (x_pref && nxt.tile == 0) load_xraw(xrA, itn);
    }
    step(bufB, xrB, cur, itc, nxt.chunk != cur.chunk);
    if (!more) break;
    cur = nxt;
    itc = itn;
  }
}

}  // namespace kxg
