// kx_rng.h -- stateless counter-based generator for the synthetic tensors.
//
// value = f(seed, tensor id, element index): any tile of any tensor can be
// regenerated anywhere (device fill kernels, host code) without holding the
// tensor.  Integer-only up to one exact int->float conversion and one float
// multiply, so host and device agree bit for bit.
//
// The reference loads a real checkpoint through uGDS (src/kimi_exec.cu:608-649);
// this build replaces that with seeded random-init weights.
#pragma once
#include <stdint.h>
#include "kx_math.h"

KX_HD uint64_t kx_mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
// per-tensor key
KX_HD uint64_t kx_rng_key(uint64_t seed, uint64_t tensor_id) {
  return kx_mix64(seed * 0x9E3779B97F4A7C15ull + tensor_id + 1ull);
}
// i-th 64-bit draw of a tensor
KX_HD uint64_t kx_rng_u64(uint64_t key, uint64_t i) {
  return kx_mix64(key + (i + 1ull) * 0x9E3779B97F4A7C15ull);
}
// i-th 32-bit word: two per 64-bit draw, low half first
KX_HD uint32_t kx_rng_u32(uint64_t key, uint64_t i) {
  return (uint32_t)(kx_rng_u64(key, i >> 1) >> (32u * (uint32_t)(i & 1ull)));
}
// approximately N(0,1): sum of twelve 16-bit uniforms, centred, scaled by 2^-16.
// Returns the centred integer sum S - 6*65535 (in [-393210, 393210]).
KX_HD int32_t kx_rng_normal_int(uint64_t key, uint64_t i) {
  uint32_t s = 0;
  for (int j = 0; j < 3; ++j) {
    uint64_t h = kx_rng_u64(key, 3ull * i + (uint64_t)j);
    s += (uint32_t)(h & 0xffffull) + (uint32_t)((h >> 16) & 0xffffull) +
         (uint32_t)((h >> 32) & 0xffffull) + (uint32_t)(h >> 48);
  }
  return (int32_t)s - 393210;
}
// sigma * z as f32: one exact conversion, one multiply by (sigma * 2^-16)
KX_HD float kx_rng_normal_f32(uint64_t key, uint64_t i, float sigma) {
  return (float)kx_rng_normal_int(key, i) * (sigma * 1.52587890625e-05f);
}
// the same, rounded to bf16; absval != 0 takes the magnitude (INT4 group scales)
KX_HD uint16_t kx_rng_normal_bf16(uint64_t key, uint64_t i, float sigma, int absval) {
  uint16_t h = kx_bf16_rne(kx_rng_normal_f32(key, i, sigma));
  return absval ? (uint16_t)(h & 0x7fffu) : h;
}
