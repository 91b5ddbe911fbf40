// kx_wave.h -- cross-lane building blocks of the gfx950 kernels (wave64).
//
// fp32 sums over lanes always follow the xor-butterfly tree (32, 16, 8, 4, 2, 1; a
// half-wave starts at 16): at each level lane l adds the value of lane l ^ m.  Because
// fp32 addition commutes, every lane of a full butterfly ends with the same bits, so the
// reductions below may compute each level in only the lanes whose result is used and
// still produce exactly the butterfly's value.  A scalar program reproduces it with
//   for m in (W/2 .. 1): for l: q[l] = p[l] + p[l ^ m]; p = q.
//
// Levels 32 and 16 use v_permlane32_swap / v_permlane16_swap (gfx950), level 8 a DPP
// rotate by 8 inside the 16-lane row, levels 4, 2, 1 DPP row shifts.
#pragma once
#include <hip/hip_runtime.h>

namespace kxw {

constexpr int DPP_QUAD_XOR1 = 0xB1, DPP_QUAD_XOR2 = 0x4E, DPP_ROW_SHL1 = 0x101, DPP_ROW_SHL2 = 0x102,
              DPP_ROW_SHL4 = 0x104, DPP_ROW_ROR8 = 0x128, DPP_ROW_MIRROR = 0x140, DPP_ROW_HALF_MIRROR = 0x141,
              DPP_ROW_BCAST15 = 0x142, DPP_ROW_BCAST31 = 0x143;

// value of the lane the control selects; 0 where the control reads outside the row
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// lanes outside ROW_MASK keep their own value
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ int dpp_keep_i(int v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, ROW_MASK, 0xf, false);
}

// lanes 32..63 of a <-> lanes 0..31 of b
__device__ __forceinline__ void swap_halves32(float &a, float &b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
// rows 1,3 of a <-> rows 0,2 of b (a row is 16 lanes)
__device__ __forceinline__ void swap_rows16(float &a, float &b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}

// Butterfly sums of NV per-lane values over W = 64 (whole wave) or 32 (each half-wave)
// lanes.  While more than one value is left, a level keeps only the half of the values
// whose index bit matches the lane's bit, so each level costs half the exchanges.
// After the call the totals sit in v[0 .. reduce_out<NV,W>()-1] of the lanes for which
// reduce_writer<NV,W>(lane) holds; reduce_index<NV,W>(lane, j) names the value in v[j].
template <int NV, int W>
struct Red {
  static_assert(NV == 1 || NV == 2 || NV == 4 || NV == 8 || NV == 16, "values per reduction");
  static_assert(W == 64 || W == 32, "reduction width");
  static constexpr int N0 = NV;
  static constexpr int N1 = (W == 64 && N0 >= 2) ? N0 / 2 : N0;   // after level 32
  static constexpr int N2 = N1 >= 2 ? N1 / 2 : N1;                // after level 16
  static constexpr int N3 = N2 >= 2 ? N2 / 2 : N2;                // after level 8
  static constexpr bool T32 = W == 64 && N0 >= 2, T16 = N1 >= 2, T8 = N2 >= 2;
};

template <int NV, int W>
__device__ __forceinline__ void reduce(float (&v)[NV], int lane) {
  using R = Red<NV, W>;
  if constexpr (W == 64) {
    if constexpr (R::T32) {
#pragma unroll
      for (int i = 0; i < R::N1; ++i) { swap_halves32(v[i], v[i + R::N1]); v[i] = v[i] + v[i + R::N1]; }
    } else {
      float t = v[0];
      swap_halves32(v[0], t);
      v[0] = v[0] + t;
    }
  }
  if constexpr (R::T16) {
#pragma unroll
    for (int i = 0; i < R::N2; ++i) { swap_rows16(v[i], v[i + R::N2]); v[i] = v[i] + v[i + R::N2]; }
  } else {
    float t = v[0];
    swap_rows16(v[0], t);
    v[0] = v[0] + t;
  }
  if constexpr (R::T8) {
    const bool hi = (lane & 8) != 0;
#pragma unroll
    for (int i = 0; i < R::N3; ++i) {
      float send = hi ? v[i] : v[i + R::N3];
      float mine = hi ? v[i + R::N3] : v[i];
      v[i] = mine + dpp_f<DPP_ROW_ROR8>(send);
    }
  } else {
    v[0] = v[0] + dpp_f<DPP_ROW_ROR8>(v[0]);
  }
#pragma unroll
  for (int i = 0; i < R::N3; ++i) {
    v[i] = v[i] + dpp_f<DPP_ROW_SHL4>(v[i]);
    v[i] = v[i] + dpp_f<DPP_ROW_SHL2>(v[i]);
    v[i] = v[i] + dpp_f<DPP_ROW_SHL1>(v[i]);
  }
}
template <int NV, int W>
__device__ __forceinline__ constexpr int reduce_out() { return Red<NV, W>::N3; }
template <int NV, int W>
__device__ __forceinline__ bool reduce_writer(int lane) {
  using R = Red<NV, W>;
  bool ok = (lane & 7) == 0;
  if (W == 64 && !R::T32) ok = ok && (lane & 32) == 0;
  if (!R::T16) ok = ok && (lane & 16) == 0;
  if (!R::T8) ok = ok && (lane & 8) == 0;
  return ok;
}
template <int NV, int W>
__device__ __forceinline__ int reduce_index(int lane, int j) {
  using R = Red<NV, W>;
  int idx = j;
  if (R::T32) idx += ((lane >> 5) & 1) * R::N1;
  if (R::T16) idx += ((lane >> 4) & 1) * R::N2;
  if (R::T8) idx += ((lane >> 3) & 1) * R::N3;
  return idx;
}

// exact wave-wide max / min (no rounding, order free); the result is wave-uniform
__device__ __forceinline__ float wave_max_f32(float v) {
#define KXW_STEP(C, M) v = fmaxf(v, __builtin_bit_cast(float, dpp_keep_i<C, M>(__builtin_bit_cast(int, v))))
  KXW_STEP(DPP_QUAD_XOR1, 0xf); KXW_STEP(DPP_QUAD_XOR2, 0xf); KXW_STEP(DPP_ROW_HALF_MIRROR, 0xf);
  KXW_STEP(DPP_ROW_MIRROR, 0xf); KXW_STEP(DPP_ROW_BCAST15, 0xa); KXW_STEP(DPP_ROW_BCAST31, 0xc);
#undef KXW_STEP
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ int wave_min_i32(int v) {
#define KXW_STEP(C, M) v = min(v, dpp_keep_i<C, M>(v))
  KXW_STEP(DPP_QUAD_XOR1, 0xf); KXW_STEP(DPP_QUAD_XOR2, 0xf); KXW_STEP(DPP_ROW_HALF_MIRROR, 0xf);
  KXW_STEP(DPP_ROW_MIRROR, 0xf); KXW_STEP(DPP_ROW_BCAST15, 0xa); KXW_STEP(DPP_ROW_BCAST31, 0xc);
#undef KXW_STEP
  return __builtin_amdgcn_readlane(v, 63);
}

}  // namespace kxw
