// kx_math.h -- scalar arithmetic shared by the host code and the gfx950 kernels.
//
// Every function here is built from IEEE-754 binary32 +, *, /, sqrt, fma,
// round-to-nearest-even and integer operations only, so a host compiler and
// hipcc (both with -ffp-contract=off) produce the same bits for the same
// input.  The reference evaluates expf/rsqrtf with the CUDA device library
// (src/kimi_exec.cu:255, :268, :379, :451); those are not reproducible off an
// NVIDIA GPU, so the path fixes its own definitions here and keeps the
// reference's rounding points around them.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define KX_HD __host__ __device__ __forceinline__
#else
#define KX_HD inline
#endif

// ---- bf16 <-> f32 (reference: bf() at src/kimi_exec.cu:240-241) -------------
KX_HD uint32_t kx_f32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
KX_HD float kx_bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }

// round-to-nearest-even f32 -> bf16 bit pattern (NaN stays a quiet NaN)
KX_HD uint16_t kx_bf16_rne(float f) {
  uint32_t u = kx_f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
KX_HD float kx_bf16_f32(uint16_t h) { return kx_bits_f32((uint32_t)h << 16); }
// bf(x): round an f32 to the nearest bf16 and widen it again
KX_HD float kx_bfround(float f) { return kx_bf16_f32(kx_bf16_rne(f)); }

// ---- exp ----------------------------------------------------------------------
// exp(x) = 2^n * p(r), n = rint(x*log2(e)), r = x - n*ln2 in two fma steps,
// p = degree-6 polynomial evaluated by Horner with fma.  About 1 ulp.
KX_HD float kx_pow2i(int n) {  // 2^n for n in [-126, 127]
  return kx_bits_f32((uint32_t)(n + 127) << 23);
}
KX_HD float kx_expf(float x) {
  if (!(x > -104.0f)) return 0.0f;                            // also catches NaN -> 0
  if (x > 88.75f) return kx_bits_f32(0x7f800000u);          // +inf
  float t = x * 1.44269504088896341f;
  float n = __builtin_rintf(t);
  float r = __builtin_fmaf(n, -0.693359375f, x);
  r = __builtin_fmaf(n, 2.12194440e-4f, r);
  float y = 1.9875691500e-4f;
  y = __builtin_fmaf(y, r, 1.3981999507e-3f);
  y = __builtin_fmaf(y, r, 8.3334519073e-3f);
  y = __builtin_fmaf(y, r, 4.1665795894e-2f);
  y = __builtin_fmaf(y, r, 1.6666665459e-1f);
  y = __builtin_fmaf(y, r, 5.0000001201e-1f);
  float z = r * r;
  y = __builtin_fmaf(y, z, r);
  y = y + 1.0f;
  int ni = (int)n;                    // |n| <= 151, exact
  int n1 = ni / 2, n2 = ni - n1;      // both within [-76, 76]
  return (y * kx_pow2i(n1)) * kx_pow2i(n2);
}

// sigmoid and SiLU with a true division (reference: :379 and :255)
KX_HD float kx_sigmoidf(float x) { return 1.0f / (1.0f + kx_expf(-x)); }
KX_HD float kx_siluf(float a) { return a / (1.0f + kx_expf(-a)); }
// 1/sqrt(v) as a correctly rounded sqrt followed by a correctly rounded divide
KX_HD float kx_rsqrtf(float v) { return 1.0f / __builtin_sqrtf(v); }

// SwiGLU mid value: bf(bf(silu(g)) * u), g and u already bf16-valued (reference :255)
KX_HD float kx_swiglu(float g, float u) { return kx_bfround(kx_bfround(kx_siluf(g)) * u); }
