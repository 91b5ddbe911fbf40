// kx_oracle.cpp -- CPU restatement of blok's kimi_exec forward hot path.
//
// TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
// calls this file; only tests/, __graft_entry__.smoke() and the cpu_baseline
// leg of bench.py do, and only as the checker or the timed CPU baseline.
//
// Every function restates a kernel or host function of the reference,
// /root/reference/src/kimi_exec.cu (cited per function as :line), in plain
// scalar C++ on host arrays.  bf16 tensors are uint16_t bit patterns.
//
// Two schedules, selected by `mode`:
//   mode 0 ("reference"): the reference's own arithmetic and summation order --
//     thread-strided partial sums over 256 virtual threads followed by the
//     shared-memory tree from d=128 (:261-267 pattern), per-weight
//     w = bf(q*scale) (:312), libm expf.  `v += a*b` is evaluated as one fmaf,
//     which is what nvcc's default -fmad=true makes of it; CUDA's expf/rsqrtf
//     are replaced by libm expf and 1/sqrtf (not reproducible off-GPU).
//   mode 1 ("kx"): the summation order and the exp() definition of the gfx950
//     kernels, so that results can be compared bit for bit and greedy tokens
//     can be required to be identical.  Both modes share every rounding point
//     of the reference (where bf() is applied).
//
// Pinning (what each function is checked against, in tests/test_oracle_*.py):
//   unpack: closed form, pack(unpack(w)) == w, all nibble/lane combinations.
//   dequant: integer-arithmetic RNE, exhaustive over 16 nibbles x 65536 scales.
//   gemv (both modes): float64 dot product of the bit-exact dequantized weights;
//     x = e_k reads back one weight, scales = 1 and x = 1 gives row sums of q.
//   rmsnorm: float64 textbook; router: sort-based top-k incl. constructed ties,
//     sum of weights == routed scale; bucket: counting-sort invariants;
//   exp (mode 1): against libm within 2 ulp over a dense sweep.
//   rope_apply: position 0 is the (2p, 2p+1) -> (p, half+p) permutation, per-pair norms are kept,
//     q.k of two rotated vectors depends on the distance of their positions only, and a float64
//     rotation in the half-split convention of the DeepSeek-V3 model code agrees.
//   model_step (the wiring of run(), :801-884): a float64 numpy forward pass of the same stack written
//     from the textbook formulation (tests/witness.py: full causal attention over the prompt, expanded
//     K/V, no cache) agrees on cache rows, hidden state and logits, and stops agreeing when a norm
//     weight is swapped, a residual add dropped, the rope dims normed, W_UK/W_UV swapped, the sine sign
//     or the pair layout changed; the DeepseekV3 model of the transformers library, given the same
//     weights, agrees as well (tests/test_oracle_wiring.py).
// No function of the hot path is pinned by a golden vector of the reference:
// the reference holds none for arithmetic (its only test, scripts/test_host.py,
// pins the argv/JSON boundary).
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <algorithm>
#include <functional>
#include <map>
#include <memory>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

extern "C" {

// ---------------------------------------------------------------------------------
// scalar helpers
// ---------------------------------------------------------------------------------
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

// bf(): round to nearest even bf16 (:240-241)
static inline uint16_t bf16_bits(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static inline float bf16_val(uint16_t h) { return u2f((uint32_t)h << 16); }
static inline float bf(float f) { return bf16_val(bf16_bits(f)); }

// exp as the gfx950 kernels define it: 2^n * p(r), Cephes-style reduction and
// degree-6 polynomial, all in fma/mul/add.
static inline float pow2i(int n) { return u2f((uint32_t)(n + 127) << 23); }
static float exp_kx(float x) {
  if (!(x > -104.0f)) return 0.0f;
  if (x > 88.75f) return INFINITY;
  float t = x * 1.44269504088896341f;
  float n = rintf(t);
  float r = fmaf(n, -0.693359375f, x);
  r = fmaf(n, 2.12194440e-4f, r);
  float y = 1.9875691500e-4f;
  y = fmaf(y, r, 1.3981999507e-3f);
  y = fmaf(y, r, 8.3334519073e-3f);
  y = fmaf(y, r, 4.1665795894e-2f);
  y = fmaf(y, r, 1.6666665459e-1f);
  y = fmaf(y, r, 5.0000001201e-1f);
  float z = r * r;
  y = fmaf(y, z, r);
  y = y + 1.0f;
  int ni = (int)n, n1 = ni / 2, n2 = ni - n1;
  return (y * pow2i(n1)) * pow2i(n2);
}
static inline float exp_m(float x, int mode) { return mode ? exp_kx(x) : expf(x); }
static inline float sigmoid_m(float x, int mode) { return 1.0f / (1.0f + exp_m(-x, mode)); }      // :379
static inline float silu_m(float a, int mode) { return a / (1.0f + exp_m(-a, mode)); }           // :255
static inline float swiglu_m(float g, float u, int mode) { return bf(bf(silu_m(g, mode)) * u); } // :255
static inline float rsqrt_o(float v) { return 1.0f / sqrtf(v); }                                   // :268

float ox_expf(float x, int mode) { return exp_m(x, mode); }
uint16_t ox_bf16(float x) { return bf16_bits(x); }

// shared-memory tree of the reference: s[t] += s[t+d], d = 128 .. 1 (:264-267)
static float tree256(float *s) {
  for (int d = 128; d; d >>= 1)
    for (int t = 0; t < d; ++t) s[t] += s[t + d];
  return s[0];
}
// xor butterfly over n lanes (n = 32 or 64): every lane adds its partner's value
static float butterfly(float *p, int n) {
  float q[64];
  for (int m = n >> 1; m; m >>= 1) {
    for (int l = 0; l < n; ++l) q[l] = p[l] + p[l ^ m];
    memcpy(p, q, sizeof(float) * n);
  }
  return p[0];
}

// ---------------------------------------------------------------------------------
// synthetic tensors: value = f(seed, tensor id, index)
// ---------------------------------------------------------------------------------
static inline uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
static inline uint64_t rng_key(uint64_t seed, uint64_t tid) { return mix64(seed * 0x9E3779B97F4A7C15ull + tid + 1ull); }
static inline uint64_t rng_u64(uint64_t key, uint64_t i) { return mix64(key + (i + 1ull) * 0x9E3779B97F4A7C15ull); }
static inline int32_t rng_normal_int(uint64_t key, uint64_t i) {
  uint32_t s = 0;
  for (int j = 0; j < 3; ++j) {
    uint64_t h = rng_u64(key, 3ull * i + j);
    s += (uint32_t)(h & 0xffff) + (uint32_t)((h >> 16) & 0xffff) + (uint32_t)((h >> 32) & 0xffff) + (uint32_t)(h >> 48);
  }
  return (int32_t)s - 393210;
}
static inline float rng_normal_f32(uint64_t key, uint64_t i, float sigma) {
  return (float)rng_normal_int(key, i) * (sigma * 1.52587890625e-05f);
}

// elements first .. first+n-1 of the tensor (a value depends on its index in the whole tensor only)
static void fill_normal_bf16_at(uint16_t *out, uint64_t first, uint64_t n, uint64_t seed, uint64_t tid, float sigma,
                                int absval) {
  uint64_t key = rng_key(seed, tid);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) {
    uint16_t h = bf16_bits(rng_normal_f32(key, first + (uint64_t)i, sigma));
    out[i] = absval ? (uint16_t)(h & 0x7fff) : h;
  }
}
void ox_fill_normal_bf16(uint16_t *out, uint64_t n, uint64_t seed, uint64_t tid, float sigma, int absval) {
  fill_normal_bf16_at(out, 0, n, seed, tid, sigma, absval);
}
// bf(mean + sigma*z): the norm weights of the random-init stack
void ox_fill_affine_bf16(uint16_t *out, uint64_t n, uint64_t seed, uint64_t tid, float mean, float sigma) {
  uint64_t key = rng_key(seed, tid);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) out[i] = bf16_bits(mean + rng_normal_f32(key, (uint64_t)i, sigma));
}
// token ids uniform in [0, vocab)
void ox_fill_tokens_u32(uint32_t *out, uint64_t n, uint64_t seed, uint64_t tid, uint32_t vocab) {
  uint64_t key = rng_key(seed, tid);
  for (uint64_t i = 0; i < n; ++i) out[i] = (uint32_t)(rng_u64(key, i) % vocab);
}
void ox_fill_normal_f32(float *out, uint64_t n, uint64_t seed, uint64_t tid, float sigma) {
  uint64_t key = rng_key(seed, tid);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) out[i] = rng_normal_f32(key, (uint64_t)i, sigma);
}
static void fill_words_u32_at(uint32_t *out, uint64_t first, uint64_t n, uint64_t seed, uint64_t tid) {
  uint64_t key = rng_key(seed, tid);
  auto word = [key](uint64_t k) { return (uint32_t)(rng_u64(key, k >> 1) >> (32u * (uint32_t)(k & 1))); };
  if ((first & 1) || (n & 1)) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)n; ++i) out[i] = word(first + (uint64_t)i);
    return;
  }
  // words 2j and 2j+1 are the two halves of one 64-bit draw
#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < (int64_t)(n >> 1); ++j) {
    uint64_t h = rng_u64(key, (first >> 1) + (uint64_t)j);
    out[2 * j] = (uint32_t)h;
    out[2 * j + 1] = (uint32_t)(h >> 32);
  }
}
void ox_fill_words_u32(uint32_t *out, uint64_t n, uint64_t seed, uint64_t tid) { fill_words_u32_at(out, 0, n, seed, tid); }

// ---------------------------------------------------------------------------------
// INT4: unpack (:309-311), dequant (:306,:312), GEMV (:300-323)
// ---------------------------------------------------------------------------------
void ox_i4_unpack(const uint32_t *packed, int8_t *q, int rows, int cols) {
  size_t words = (size_t)rows * (cols / 8);
  for (size_t i = 0; i < words; ++i)
    for (int lane = 0; lane < 8; ++lane) q[i * 8 + lane] = (int8_t)((int)((packed[i] >> (4 * lane)) & 0xf) - 8);
}

void ox_i4_dequant(const uint32_t *packed, const uint16_t *scale, uint16_t *w, int rows, int cols) {
  int groups = cols / 32, pc = cols / 8;
#pragma omp parallel for schedule(static)
  for (int r = 0; r < rows; ++r)
    for (int g = 0; g < groups; ++g) {
      float sc = bf16_val(scale[(size_t)r * groups + g]);
      for (int p = 0; p < 4; ++p) {
        uint32_t word = packed[(size_t)r * pc + g * 4 + p];
        for (int lane = 0; lane < 8; ++lane) {
          int q = (int)((word >> (4 * lane)) & 0xf) - 8;
          w[(size_t)r * cols + g * 32 + p * 8 + lane] = bf16_bits((float)q * sc);
        }
      }
    }
}

// one output row, reference schedule: thread g owns groups g, g+256, ... (:305-315)
static float i4_row_ref(const uint32_t *prow, const uint16_t *srow, const float *x, int cols) {
  float s[256];
  int groups = cols / 32;
  for (int t = 0; t < 256; ++t) {
    float v = 0;
    for (int g = t; g < groups; g += 256) {
      float sc = bf16_val(srow[g]);
      int base = g * 32;
      for (int p = 0; p < 4; ++p) {
        uint32_t word = prow[g * 4 + p];
        for (int lane = 0; lane < 8; ++lane) {
          int q = (int)((word >> (4 * lane)) & 0xf) - 8;
          v = fmaf(x[base + p * 8 + lane], bf((float)q * sc), v);
        }
      }
    }
    s[t] = v;
  }
  return tree256(s);
}

// activations of one token prepared the way the kernel keeps them: per group 32
// values in chain order (k = 8w + {0,4,1,5,2,6,3,7}), the odd nibbles' values
// divided by 16, and the start value of the chain.
struct XPrep {
  std::vector<float> v;      // [groups][32]
  std::vector<float> neg_c;  // [groups]
};
static void i4_prep_x(XPrep &xp, const uint16_t *x, int cols) {
  static const int order[8] = {0, 4, 1, 5, 2, 6, 3, 7};
  int groups = cols / 32;
  xp.v.resize((size_t)groups * 32);
  xp.neg_c.resize(groups);
  for (int g = 0; g < groups; ++g) {
    float *v = &xp.v[(size_t)g * 32];
    for (int w = 0; w < 4; ++w)
      for (int c = 0; c < 8; ++c) {
        float f = bf16_val(x[g * 32 + w * 8 + order[c]]);
        v[w * 8 + c] = (order[c] & 1) ? f * 0.0625f : f;
      }
    float c = 0.0f;
    for (int i = 0; i < 32; ++i) c = fmaf(v[i], (i & 2) ? 1152.0f : 1032.0f, c);
    xp.neg_c[g] = -c;
  }
}
// one output row, kx schedule
static float i4_row_kx(const uint32_t *prow, const uint16_t *srow, const XPrep &xp, int cols) {
  int S = cols / 1024;
  float y = 0.0f;
  for (int s = 0; s < S; ++s) {
    float p[32];
    for (int l = 0; l < 32; ++l) {
      int g = 32 * s + l;
      const float *v = &xp.v[(size_t)g * 32];
      float acc = xp.neg_c[g];
      for (int w = 0; w < 4; ++w) {
        uint32_t W = prow[g * 4 + w], W8 = W >> 8;
        float a[8] = {1024.0f + (float)(W & 0xf),  1024.0f + (float)((W >> 16) & 0xf),
                      1024.0f + (float)(W & 0xf0), 1024.0f + (float)((W >> 16) & 0xf0),
                      1024.0f + (float)(W8 & 0xf), 1024.0f + (float)((W8 >> 16) & 0xf),
                      1024.0f + (float)(W8 & 0xf0), 1024.0f + (float)((W8 >> 16) & 0xf0)};
        for (int c = 0; c < 8; ++c) acc = fmaf(a[c], v[w * 8 + c], acc);
      }
      p[l] = bf16_val(srow[g]) * acc;
    }
    float B = butterfly(p, 32);
    y = s ? y + B : B;
  }
  return y;
}

// y[t, r] = bf(sum_k x[t,k] w[r,k]); x bf16 [T, cols], y bf16 [T, rows]
void ox_i4_gemv(const uint32_t *packed, const uint16_t *scale, const uint16_t *x, uint16_t *y, int rows, int cols,
                int tokens, int mode) {
  int groups = cols / 32, pc = cols / 8;
  for (int t = 0; t < tokens; ++t) {
    std::vector<float> xf(cols);
    for (int k = 0; k < cols; ++k) xf[k] = bf16_val(x[(size_t)t * cols + k]);
    XPrep xp;
    if (mode) i4_prep_x(xp, x + (size_t)t * cols, cols);
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
      float v = mode ? i4_row_kx(packed + (size_t)r * pc, scale + (size_t)r * groups, xp, cols)
                     : i4_row_ref(packed + (size_t)r * pc, scale + (size_t)r * groups, xf.data(), cols);
      y[(size_t)t * rows + r] = bf16_bits(v);
    }
  }
}

// ---------------------------------------------------------------------------------
// RMSNorm (:258-270) and bf16 matvec (:272-298)
// ---------------------------------------------------------------------------------
static void rmsnorm_row(const uint16_t *x, const uint16_t *w, uint16_t *y, int n, float eps, int mode) {
  float total;
  if (!mode) {
    float s[256];
    for (int t = 0; t < 256; ++t) {
      float v = 0;
      for (int i = t; i < n; i += 256) { float f = bf16_val(x[i]); v = fmaf(f, f, v); }
      s[t] = v;
    }
    total = tree256(s);
  } else {
    float ws[4];
    for (int wv = 0; wv < 4; ++wv) {
      float p[64];
      for (int l = 0; l < 64; ++l) {
        int t = wv * 64 + l;
        float v = 0;
        for (int c = t; c < n / 8; c += 256)
          for (int e = 0; e < 8; ++e) { float f = bf16_val(x[c * 8 + e]); v = fmaf(f, f, v); }
        p[l] = v;
      }
      ws[wv] = butterfly(p, 64);
    }
    total = ((ws[0] + ws[1]) + ws[2]) + ws[3];
  }
  float scale = rsqrt_o(total / (float)n + eps);
  for (int i = 0; i < n; ++i) y[i] = bf16_bits(bf(bf16_val(x[i]) * scale) * bf16_val(w[i]));
}
void ox_rmsnorm(const uint16_t *x, const uint16_t *w, uint16_t *y, int tokens, int n, float eps, int mode) {
  for (int t = 0; t < tokens; ++t) rmsnorm_row(x + (size_t)t * n, w, y + (size_t)t * n, n, eps, mode);
}

static float bf16_row_dot(const uint16_t *wrow, const float *x, int cols, int mode) {
  if (!mode) {
    float s[256];
    for (int t = 0; t < 256; ++t) {
      float v = 0;
      for (int c = t; c < cols; c += 256) v = fmaf(bf16_val(wrow[c]), x[c], v);
      s[t] = v;
    }
    return tree256(s);
  }
  int S = cols / 512;
  float y = 0.0f;
  for (int s = 0; s < S; ++s) {
    float p[64];
    for (int l = 0; l < 64; ++l) {
      float acc = 0.0f;
      const uint16_t *wp = wrow + s * 512 + l * 8;
      const float *xp = x + s * 512 + l * 8;
      for (int e = 0; e < 8; ++e) acc = fmaf(bf16_val(wp[e]), xp[e], acc);
      p[l] = acc;
    }
    float B = butterfly(p, 64);
    y = s ? y + B : B;
  }
  return y;
}
// raw fp32 sums, x given as f32
static void gemv_bf16_raw(const uint16_t *w, const float *x, float *y, int rows, int cols, int mode) {
#pragma omp parallel for schedule(static)
  for (int r = 0; r < rows; ++r) y[r] = bf16_row_dot(w + (size_t)r * cols, x, cols, mode);
}
// out_f32 == 0: y bf16 [T, rows] rounded (:283); else y f32 [T, rows] unrounded (:297)
void ox_gemv_bf16(const uint16_t *w, const uint16_t *x, void *y, int rows, int cols, int tokens, int out_f32, int mode) {
  std::vector<float> xf(cols), yf(rows);
  for (int t = 0; t < tokens; ++t) {
    for (int k = 0; k < cols; ++k) xf[k] = bf16_val(x[(size_t)t * cols + k]);
    gemv_bf16_raw(w, xf.data(), yf.data(), rows, cols, mode);
    if (out_f32) memcpy((float *)y + (size_t)t * rows, yf.data(), sizeof(float) * rows);
    else for (int r = 0; r < rows; ++r) ((uint16_t *)y)[(size_t)t * rows + r] = bf16_bits(yf[r]);
  }
}

// ---------------------------------------------------------------------------------
// router (:372-397) and bucketing
// ---------------------------------------------------------------------------------
void ox_router_topk(const float *logits, const float *bias, uint16_t *ids, float *weights, int tokens, int experts,
                    int topk, float routed_scale, int mode) {
  std::vector<float> score(experts), sel(experts);
  for (int t = 0; t < tokens; ++t) {
    for (int e = 0; e < experts; ++e) {
      score[e] = sigmoid_m(logits[(size_t)t * experts + e], mode);
      sel[e] = score[e] + bias[e];
    }
    float sum = 0;
    for (int k = 0; k < topk; ++k) {
      int id = 0;
      float best = -INFINITY;
      for (int i = 0; i < experts; ++i)
        if (sel[i] > best) best = sel[i], id = i;
      ids[(size_t)t * topk + k] = (uint16_t)id;
      weights[(size_t)t * topk + k] = score[id];
      sum += score[id];
      sel[id] = -INFINITY;
    }
    for (int k = 0; k < topk; ++k)
      weights[(size_t)t * topk + k] = weights[(size_t)t * topk + k] / (sum + 1.0e-20f) * routed_scale;
  }
}

// pairs = token*topk+slot sorted by (expert, token, slot); returns the number of active experts
int ox_bucket(const uint16_t *ids, int tokens, int experts, int topk, int *counts, int *offsets, int *pairs, int *active) {
  int n = tokens * topk;
  for (int e = 0; e < experts; ++e) counts[e] = 0;
  for (int p = 0; p < n; ++p) counts[ids[p]]++;
  int run = 0, na = 0;
  for (int e = 0; e < experts; ++e) {
    offsets[e] = run;
    if (counts[e] > 0) active[na++] = e;
    run += counts[e];
  }
  offsets[experts] = run;
  std::vector<int> pos(offsets, offsets + experts);
  for (int p = 0; p < n; ++p) pairs[pos[ids[p]]++] = p;
  return na;
}

// ---------------------------------------------------------------------------------
// one routed-MoE decode layer: the MoE branch of run() (:835-877)
// ---------------------------------------------------------------------------------
struct ox_moe_weights {
  const uint16_t *router_gate;  // bf16 [E, hidden]
  const float *router_bias;     // f32 [E]
  const uint32_t *gate_packed; const uint16_t *gate_scale;
  const uint32_t *up_packed;   const uint16_t *up_scale;
  const uint32_t *down_packed; const uint16_t *down_scale;
  const uint16_t *shared_gate, *shared_up, *shared_down;
};

// n bf16 [T, hidden] (FFN input), x bf16 [T, hidden] residual stream, updated in place unless flags&1
// (then `down` is written).  Optional outputs (may be null): logits f32 [T,E], ids u16 [T,topk],
// weights f32 [T,topk], mid bf16 [T*topk, moe_inter], eout bf16 [T*topk, hidden].
void ox_moe_layer(const ox_moe_weights *w, const uint16_t *n, uint16_t *x, int tokens, int hidden, int moe_inter,
                  int shared_inter, int experts, int topk, float routed_scale, uint32_t flags, int mode,
                  float *o_logits, uint16_t *o_ids, float *o_weights, uint16_t *o_mid, uint16_t *o_eout);
// the six tensors of one routed expert: packed i32 [N, K/8] and scales bf16 [N, K/32] per projection
struct ExpertView {
  const uint32_t *gate_p; const uint16_t *gate_s;
  const uint32_t *up_p;   const uint16_t *up_s;
  const uint32_t *down_p; const uint16_t *down_s;
};
// Where a layer's routed experts come from.  A null source reads them at expert * stride of the tensors in
// ox_moe_weights; the decoder stack can pass one that produces an expert when it is first selected (a view is
// only used until the next one is asked for).
typedef std::function<ExpertView(int)> ExpertSource;
static void moe_layer_impl(const ox_moe_weights *w, const uint16_t *n, uint16_t *x, int tokens, int hidden, int moe_inter,
                           int shared_inter, int experts, int topk, float routed_scale, uint32_t flags, int mode,
                           float *o_logits, uint16_t *o_ids, float *o_weights, uint16_t *o_mid, uint16_t *o_eout,
                           const uint16_t *in_ids, const float *in_weights, const ExpertSource *source = nullptr) {
  const int H = hidden, I = moe_inter, SI = shared_inter, E = experts, K = topk;
  std::vector<float> logits((size_t)tokens * E), weights((size_t)tokens * K);
  std::vector<uint16_t> ids((size_t)tokens * K);
  if (in_ids) {  // routing decided elsewhere (checked separately): only the expert arithmetic is restated
    memcpy(ids.data(), in_ids, ids.size() * 2);
    memcpy(weights.data(), in_weights, weights.size() * 4);
  } else {
    ox_gemv_bf16(w->router_gate, n, logits.data(), E, H, tokens, 1, mode);  // :838
    ox_router_topk(logits.data(), w->router_bias, ids.data(), weights.data(), tokens, E, K, routed_scale, mode);
  }
  if (o_logits) memcpy(o_logits, logits.data(), logits.size() * 4);
  if (o_ids) memcpy(o_ids, ids.data(), ids.size() * 2);
  if (o_weights) memcpy(o_weights, weights.data(), weights.size() * 4);
  std::vector<uint16_t> g(I), u(I), mid(I), y(H), sg(SI), su(SI), smid(SI), sy(H);
  for (int t = 0; t < tokens; ++t) {
    const uint16_t *nt = n + (size_t)t * H;
    std::vector<float> down(H, 0.0f);
    for (int slot = 0; slot < K; ++slot) {  // :845-870
      int e = ids[(size_t)t * K + slot];
      ExpertView v;
      if (source) {
        v = (*source)(e);
      } else {
        size_t wo = (size_t)e * I * (H / 8), so = (size_t)e * I * (H / 32);
        v = {w->gate_packed + wo, w->gate_scale + so, w->up_packed + wo, w->up_scale + so, w->down_packed + wo,
             w->down_scale + so};
      }
      ox_i4_gemv(v.gate_p, v.gate_s, nt, g.data(), I, H, 1, mode);
      ox_i4_gemv(v.up_p, v.up_s, nt, u.data(), I, H, 1, mode);
      for (int r = 0; r < I; ++r) mid[r] = bf16_bits(swiglu_m(bf16_val(g[r]), bf16_val(u[r]), mode));
      ox_i4_gemv(v.down_p, v.down_s, mid.data(), y.data(), H, I, 1, mode);
      float wk = weights[(size_t)t * K + slot];
      for (int r = 0; r < H; ++r) down[r] = fmaf(bf16_val(y[r]), wk, down[r]);  // :401
      if (o_mid) memcpy(o_mid + ((size_t)t * K + slot) * I, mid.data(), (size_t)I * 2);
      if (o_eout) memcpy(o_eout + ((size_t)t * K + slot) * H, y.data(), (size_t)H * 2);
    }
    for (int r = 0; r < H; ++r) down[r] = bf(down[r]);  // :871
    // shared expert through bf16_mlp (:674-686): down = bf(down + bf(W_d mid))
    ox_gemv_bf16(w->shared_gate, nt, sg.data(), SI, H, 1, 0, mode);
    ox_gemv_bf16(w->shared_up, nt, su.data(), SI, H, 1, 0, mode);
    for (int r = 0; r < SI; ++r) smid[r] = bf16_bits(swiglu_m(bf16_val(sg[r]), bf16_val(su[r]), mode));
    ox_gemv_bf16(w->shared_down, smid.data(), sy.data(), H, SI, 1, 0, mode);
    for (int r = 0; r < H; ++r) {
      float d = bf(down[r] + bf16_val(sy[r]));
      uint16_t *xr = x + (size_t)t * H + r;
      *xr = (flags & 1u) ? bf16_bits(d) : bf16_bits(bf16_val(*xr) + d);  // :877
    }
  }
}

// ---------------------------------------------------------------------------------
// RoPE / YaRN tables (:325-357) and the softmax scale (:428-429)
// ---------------------------------------------------------------------------------
struct ox_config {  // same layout as kx_config (include/kx.h)
  int32_t n_layers, first_dense, hidden, heads, qk_nope, qk_rope, v_head, q_rank, kv_rank, experts, topk,
      moe_inter, shared_inter, dense_inter, vocab, max_batch, max_context;
  uint32_t eos_id;
  float rms_eps, rope_theta, routed_scale, yarn_factor, yarn_beta_fast, yarn_beta_slow, yarn_orig_ctx,
      yarn_mscale_all_dim, init_sigma, expert_scale_sigma;
  uint64_t seed;
};

static float yarn_correction_dim(const ox_config *c, float rotations, float dim) {  // :325-327
  volatile float two_pi = 2.0f * 3.14159265358979323846f;
  return dim * logf(c->yarn_orig_ctx / (rotations * two_pi)) / (2.0f * logf(c->rope_theta));
}
static float yarn_ramp(float low, float high, float at) {  // :329-332
  if (low == high) high += 0.001f;
  return fminf(1.0f, fmaxf(0.0f, (at - low) / (high - low)));
}
float ox_yarn_inv_freq(const ox_config *c, int pair) {  // :334-344
  float dim = (float)c->qk_rope;
  float freq_extra = powf(c->rope_theta, -2.0f * (float)pair / dim);
  float freq_inter = freq_extra / c->yarn_factor;
  float low = floorf(yarn_correction_dim(c, c->yarn_beta_fast, dim));
  float high = ceilf(yarn_correction_dim(c, c->yarn_beta_slow, dim));
  low = fmaxf(low, 0.0f);
  high = fminf(high, dim - 1.0f);
  float inv_freq_mask = 1.0f - yarn_ramp(low, high, (float)pair);
  return freq_inter * (1.0f - inv_freq_mask) + freq_extra * inv_freq_mask;
}
// table row of a position: qk_rope/2 cosines then qk_rope/2 sines, rounded to bf16 (:351)
void ox_rope_table(const ox_config *c, int pos0, int n, uint16_t *out) {
  int half = c->qk_rope / 2;
  for (int i = 0; i < n; ++i)
    for (int p = 0; p < half; ++p) {
      float freq = ox_yarn_inv_freq(c, p);
      float ang = (float)(pos0 + i) * freq;
      out[(size_t)i * c->qk_rope + p] = bf16_bits(cosf(ang));
      out[(size_t)i * c->qk_rope + half + p] = bf16_bits(sinf(ang));
    }
}
// the two factors of the score scale: rsqrt(qk_nope+qk_rope) and mscale (:428-429)
void ox_softmax_scale(const ox_config *c, float *rs, float *mscale) {
  *rs = rsqrt_o((float)(c->qk_nope + c->qk_rope));
  *mscale = 0.1f * c->yarn_mscale_all_dim * logf(c->yarn_factor) + 1.0f;
}
// interleaved-pair rotation: reads (2p, 2p+1), writes (p, half+p) (:352-356); x, y f32 of bf16 values
static void rope_apply(const float *x, float *y, const uint16_t *tab, int rotary) {
  int half = rotary / 2;
  for (int p = 0; p < half; ++p) {
    float c = bf16_val(tab[p]), s = bf16_val(tab[half + p]);
    float x0 = x[2 * p], x1 = x[2 * p + 1];
    y[p] = bf(bf(x0 * c) - bf(x1 * s));
    y[half + p] = bf(bf(x1 * c) + bf(x0 * s));
  }
}
// rope_apply for the tests: x, y f32 [rotary] (bf16 values), tab = one row of ox_rope_table
void ox_rope_apply(const float *x, float *y, const uint16_t *tab, int rotary) { rope_apply(x, y, tab, rotary); }

// ---------------------------------------------------------------------------------
// The decoder stack: run() / generate() (:780-893)
// ---------------------------------------------------------------------------------
enum {  // tensor ids: global tensors use the id itself, layer L uses (L+1)*64 + id
  TID_EMBED = 1, TID_FINAL_NORM = 2, TID_LM_HEAD = 3, TID_PROMPT = 4,
  TL_INPUT_LN = 0, TL_QA = 1, TL_QA_LN = 2, TL_QB = 3, TL_KVA = 4, TL_KV_LN = 5, TL_KVB = 6, TL_O = 7, TL_POST_LN = 8,
  TL_DENSE_GATE = 9, TL_DENSE_UP = 10, TL_DENSE_DOWN = 11, TL_ROUTER = 12, TL_ROUTER_BIAS = 13,
  TL_GATE_P = 14, TL_GATE_S = 15, TL_UP_P = 16, TL_UP_S = 17, TL_DOWN_P = 18, TL_DOWN_S = 19,
  TL_SH_GATE = 20, TL_SH_UP = 21, TL_SH_DOWN = 22
};

struct OxLayer {
  std::vector<uint16_t> input_ln, qa, qa_ln, qb, kva, kv_ln, kvb, o, post_ln;
  std::vector<uint16_t> dgate, dup, ddown;
  std::vector<uint16_t> router, gate_s, up_s, down_s, sh_gate, sh_up, sh_down;
  std::vector<float> router_bias;
  std::vector<uint32_t> gate_p, up_p, down_p;
  // a model whose experts are produced on demand keeps the ones in use here instead of in the six tensors above
  struct Expert {
    std::vector<uint32_t> gate_p, up_p, down_p;
    std::vector<uint16_t> gate_s, up_s, down_s;
    bool given = false;  // holds a tensor handed over with ox_model_set_tensor: never dropped
  };
  std::map<int, std::unique_ptr<Expert>> on_demand;
  // latent cache [B][max_context][kv_rank + qk_rope] bf16; mode 0 also keeps the expanded
  // fp32 K [B][ctx][heads*(nope+rope)] and V [B][ctx][heads*v_head] of the reference (:192-238)
  std::vector<uint16_t> latent;
  std::vector<float> K, V;
};

struct ox_model {
  ox_config c;
  int mode;
  // experts on demand: a decode step touches topk experts per layer, so the stack of BASELINE config 5 (24 layers
  // x 384 experts = 228 GB of routed tensors) needs a few GB of host memory this way.  The generator's values
  // depend on (seed, tensor, index) only, so an expert produced alone equals its part of the whole tensor.
  bool on_demand = false;
  size_t kept = 0, keep_at_most = 192;  // experts held over all layers before the ones not handed over are dropped
  uint64_t produced = 0;                // experts generated so far (for the tests)
  std::vector<std::unique_ptr<OxLayer::Expert>> spare;
  float expert_scale_sigma;
  std::vector<uint16_t> embed, final_norm, lm_head, rope_tab;
  std::vector<OxLayer> layers;
  std::vector<uint16_t> x;  // residual stream [B][hidden]
  std::vector<float> last_logits;  // [B][vocab] bf16-rounded logits of the last sampled step
};

static void fill_bf16(std::vector<uint16_t> &v, size_t n, uint64_t seed, uint64_t tid, float sigma, int absval = 0) {
  v.resize(n);
  ox_fill_normal_bf16(v.data(), n, seed, tid, sigma, absval);
}
static void fill_ln(std::vector<uint16_t> &v, size_t n, uint64_t seed, uint64_t tid) {
  v.resize(n);
  ox_fill_affine_bf16(v.data(), n, seed, tid, 1.0f, 0.02f);
}
static void fill_words(std::vector<uint32_t> &v, size_t n, uint64_t seed, uint64_t tid) {
  v.resize(n);
  ox_fill_words_u32(v.data(), n, seed, tid);
}

// flags bit 0: routed experts are produced when first selected instead of all at creation
ox_model *ox_model_create_ex(const ox_config *cfg, int mode, uint32_t flags) {
  const float expert_scale_sigma = cfg->expert_scale_sigma;
  ox_model *m = new ox_model();
  m->c = *cfg;
  m->mode = mode;
  m->on_demand = (flags & 1u) != 0;
  m->expert_scale_sigma = expert_scale_sigma;
  const ox_config &c = m->c;
  const size_t H = c.hidden, V = c.vocab, E = c.experts, I = c.moe_inter, SI = c.shared_inter, D = c.dense_inter;
  const size_t KD = (size_t)c.heads * (c.qk_nope + c.qk_rope), VD = (size_t)c.heads * c.v_head;
  const size_t KVA = c.kv_rank + c.qk_rope, KVB = (size_t)c.heads * (c.qk_nope + c.v_head);
  const float sg = c.init_sigma;
  fill_bf16(m->embed, V * H, c.seed, TID_EMBED, 1.0f);
  fill_ln(m->final_norm, H, c.seed, TID_FINAL_NORM);
  fill_bf16(m->lm_head, V * H, c.seed, TID_LM_HEAD, sg);
  m->rope_tab.resize((size_t)c.max_context * c.qk_rope);
  ox_rope_table(&c, 0, c.max_context, m->rope_tab.data());
  m->layers.resize(c.n_layers);
  for (int l = 0; l < c.n_layers; ++l) {
    OxLayer &L = m->layers[l];
    const uint64_t b = (uint64_t)(l + 1) * 64;
    fill_ln(L.input_ln, H, c.seed, b + TL_INPUT_LN);
    fill_bf16(L.qa, (size_t)c.q_rank * H, c.seed, b + TL_QA, sg);
    fill_ln(L.qa_ln, c.q_rank, c.seed, b + TL_QA_LN);
    fill_bf16(L.qb, KD * c.q_rank, c.seed, b + TL_QB, sg);
    fill_bf16(L.kva, KVA * H, c.seed, b + TL_KVA, sg);
    fill_ln(L.kv_ln, c.kv_rank, c.seed, b + TL_KV_LN);
    fill_bf16(L.kvb, KVB * c.kv_rank, c.seed, b + TL_KVB, sg);
    fill_bf16(L.o, H * VD, c.seed, b + TL_O, sg);
    fill_ln(L.post_ln, H, c.seed, b + TL_POST_LN);
    if (l < c.first_dense) {
      fill_bf16(L.dgate, D * H, c.seed, b + TL_DENSE_GATE, sg);
      fill_bf16(L.dup, D * H, c.seed, b + TL_DENSE_UP, sg);
      fill_bf16(L.ddown, H * D, c.seed, b + TL_DENSE_DOWN, sg);
    } else {
      fill_bf16(L.router, E * H, c.seed, b + TL_ROUTER, 1.0f / sqrtf((float)H));
      L.router_bias.resize(E);
      ox_fill_normal_f32(L.router_bias.data(), E, c.seed, b + TL_ROUTER_BIAS, 0.01f);
      if (!m->on_demand) {
        fill_words(L.gate_p, E * I * H / 8, c.seed, b + TL_GATE_P);
        fill_bf16(L.gate_s, E * I * H / 32, c.seed, b + TL_GATE_S, expert_scale_sigma, 1);
        fill_words(L.up_p, E * I * H / 8, c.seed, b + TL_UP_P);
        fill_bf16(L.up_s, E * I * H / 32, c.seed, b + TL_UP_S, expert_scale_sigma, 1);
        fill_words(L.down_p, E * H * I / 8, c.seed, b + TL_DOWN_P);
        fill_bf16(L.down_s, E * H * I / 32, c.seed, b + TL_DOWN_S, expert_scale_sigma, 1);
      }
      fill_bf16(L.sh_gate, SI * H, c.seed, b + TL_SH_GATE, sg);
      fill_bf16(L.sh_up, SI * H, c.seed, b + TL_SH_UP, sg);
      fill_bf16(L.sh_down, H * SI, c.seed, b + TL_SH_DOWN, sg);
    }
    L.latent.assign((size_t)c.max_batch * c.max_context * KVA, 0);
    if (!mode) {
      L.K.assign((size_t)c.max_batch * c.max_context * KD, 0.0f);
      L.V.assign((size_t)c.max_batch * c.max_context * VD, 0.0f);
    }
  }
  m->x.assign((size_t)c.max_batch * H, 0);
  m->last_logits.assign((size_t)c.max_batch * V, 0.0f);
  return m;
}
ox_model *ox_model_create(const ox_config *cfg, int mode) { return ox_model_create_ex(cfg, mode, 0); }
void ox_model_destroy(ox_model *m) { delete m; }
uint64_t ox_model_experts_produced(const ox_model *m) { return m->produced; }
// how many on-demand experts are held before the ones that can be produced again are dropped (at least 1)
void ox_model_keep_experts(ox_model *m, int n) { m->keep_at_most = n < 1 ? 1 : (size_t)n; }

// expert e of layer l of a model that produces its experts on demand.  Dropped experts go to a list of spares and
// their buffers are filled again for the next expert: fresh pages cost more than the values that go into them.
static OxLayer::Expert &expert_on_demand(ox_model *m, int l, int e) {
  OxLayer &L = m->layers[l];
  auto it = L.on_demand.find(e);
  if (it != L.on_demand.end()) return *it->second;
  if (m->kept >= m->keep_at_most) {  // drop every expert that can be produced again
    m->kept = 0;
    for (OxLayer &o : m->layers)
      for (auto j = o.on_demand.begin(); j != o.on_demand.end();) {
        if (j->second->given) {
          ++j, ++m->kept;
        } else {
          m->spare.push_back(std::move(j->second));
          j = o.on_demand.erase(j);
        }
      }
  }
  std::unique_ptr<OxLayer::Expert> &slot = L.on_demand[e];
  if (m->spare.empty()) {
    slot.reset(new OxLayer::Expert());
  } else {
    slot = std::move(m->spare.back());
    m->spare.pop_back();
  }
  OxLayer::Expert &x = *slot;
  const ox_config &c = m->c;
  const uint64_t b = (uint64_t)(l + 1) * 64, words = (uint64_t)c.moe_inter * c.hidden / 8, scales = words / 4;
  x.gate_p.resize(words); x.up_p.resize(words); x.down_p.resize(words);
  x.gate_s.resize(scales); x.up_s.resize(scales); x.down_s.resize(scales);
  fill_words_u32_at(x.gate_p.data(), e * words, words, c.seed, b + TL_GATE_P);
  fill_normal_bf16_at(x.gate_s.data(), e * scales, scales, c.seed, b + TL_GATE_S, m->expert_scale_sigma, 1);
  fill_words_u32_at(x.up_p.data(), e * words, words, c.seed, b + TL_UP_P);
  fill_normal_bf16_at(x.up_s.data(), e * scales, scales, c.seed, b + TL_UP_S, m->expert_scale_sigma, 1);
  fill_words_u32_at(x.down_p.data(), e * words, words, c.seed, b + TL_DOWN_P);
  fill_normal_bf16_at(x.down_s.data(), e * scales, scales, c.seed, b + TL_DOWN_S, m->expert_scale_sigma, 1);
  ++m->kept;
  ++m->produced;
  return x;
}

// Overwrites one weight tensor of the model with `bytes` bytes from `src` (the element type the model keeps:
// bf16, u32 words, f32 for the router bias).  layer < 0: id is TID_EMBED / TID_FINAL_NORM / TID_LM_HEAD; else a
// TL_* id; expert >= 0 addresses one expert's part of a routed tensor.  Returns 0, or -1 when the id, the
// coordinates or the byte count do not fit.  It is how a test hands the oracle the weights of a checkpoint
// (the reference reads them per tile, load_tensor / load_rows, :608-649).
int ox_model_set_tensor(ox_model *m, int layer, int id, int expert, const void *src, uint64_t bytes) {
  void *dst = nullptr;
  size_t have = 0;
  auto whole16 = [&](std::vector<uint16_t> &v) { dst = v.data(); have = v.size() * 2; };
  auto part = [&](auto &v, size_t esz) {
    const size_t per = v.size() / (size_t)m->c.experts;
    if (expert < 0 || expert >= m->c.experts) return;
    dst = v.data() + per * (size_t)expert;
    have = per * esz;
  };
  if (m->on_demand && layer >= m->c.first_dense && layer < m->c.n_layers && id >= TL_GATE_P && id <= TL_DOWN_S) {
    if (expert < 0 || expert >= m->c.experts) return -1;
    OxLayer::Expert &x = expert_on_demand(m, layer, expert);
    x.given = true;
    switch (id) {
      case TL_GATE_P: dst = x.gate_p.data(); have = x.gate_p.size() * 4; break;
      case TL_GATE_S: dst = x.gate_s.data(); have = x.gate_s.size() * 2; break;
      case TL_UP_P: dst = x.up_p.data(); have = x.up_p.size() * 4; break;
      case TL_UP_S: dst = x.up_s.data(); have = x.up_s.size() * 2; break;
      case TL_DOWN_P: dst = x.down_p.data(); have = x.down_p.size() * 4; break;
      default: dst = x.down_s.data(); have = x.down_s.size() * 2; break;
    }
    if (have != bytes) return -1;
    memcpy(dst, src, bytes);
    return 0;
  }
  if (layer < 0) {
    if (id == TID_EMBED) whole16(m->embed);
    else if (id == TID_FINAL_NORM) whole16(m->final_norm);
    else if (id == TID_LM_HEAD) whole16(m->lm_head);
  } else if (layer < m->c.n_layers) {
    OxLayer &L = m->layers[layer];
    switch (id) {
      case TL_INPUT_LN: whole16(L.input_ln); break;
      case TL_QA: whole16(L.qa); break;
      case TL_QA_LN: whole16(L.qa_ln); break;
      case TL_QB: whole16(L.qb); break;
      case TL_KVA: whole16(L.kva); break;
      case TL_KV_LN: whole16(L.kv_ln); break;
      case TL_KVB: whole16(L.kvb); break;
      case TL_O: whole16(L.o); break;
      case TL_POST_LN: whole16(L.post_ln); break;
      case TL_DENSE_GATE: whole16(L.dgate); break;
      case TL_DENSE_UP: whole16(L.dup); break;
      case TL_DENSE_DOWN: whole16(L.ddown); break;
      case TL_ROUTER: whole16(L.router); break;
      case TL_ROUTER_BIAS: dst = L.router_bias.data(); have = L.router_bias.size() * 4; break;
      case TL_GATE_P: part(L.gate_p, 4); break;
      case TL_GATE_S: part(L.gate_s, 2); break;
      case TL_UP_P: part(L.up_p, 4); break;
      case TL_UP_S: part(L.up_s, 2); break;
      case TL_DOWN_P: part(L.down_p, 4); break;
      case TL_DOWN_S: part(L.down_s, 2); break;
      case TL_SH_GATE: whole16(L.sh_gate); break;
      case TL_SH_UP: whole16(L.sh_up); break;
      case TL_SH_DOWN: whole16(L.sh_down); break;
      default: break;
    }
  }
  if (!dst || have == 0 || have != bytes) return -1;
  memcpy(dst, src, bytes);
  return 0;
}

// y = bf(W x) for one token through the selected schedule
static void mv(const ox_model *m, const std::vector<uint16_t> &w, const uint16_t *x, uint16_t *y, int rows, int cols) {
  ox_gemv_bf16(w.data(), x, y, rows, cols, 1, 0, m->mode);
}

// softmax + PV of the reference over the expanded fp32 K/V of one sequence (:692-716), 64-position tiles
static void attn_ref(const ox_model *m, const OxLayer &L, int b, int seq, const float *q_rot, uint16_t *out) {
  const ox_config &c = m->c;
  const int QK = c.qk_nope + c.qk_rope, KD = c.heads * QK, VD = c.heads * c.v_head;
  float rs, ms;
  ox_softmax_scale(&c, &rs, &ms);
  const float *Kb = &L.K[(size_t)b * c.max_context * KD], *Vb = &L.V[(size_t)b * c.max_context * VD];
#pragma omp parallel for schedule(static)
  for (int h = 0; h < c.heads; ++h) {
    std::vector<float> sc(seq);
    for (int t = 0; t < seq; ++t) {  // attn_tile_score_k (:414-431)
      float s[256];
      for (int i = 0; i < 256; ++i) {
        float v = 0;
        for (int j = i; j < QK; j += 256) v = fmaf(q_rot[h * QK + j], Kb[(size_t)t * KD + h * QK + j], v);
        s[i] = v;
      }
      sc[t] = bf(bf(tree256(s)) * rs * ms * ms);
    }
    float mx = -INFINITY;
    for (int t = 0; t < seq; ++t) mx = fmaxf(mx, sc[t]);  // :433-445
    float sum = 0;
    for (int start = 0; start < seq; start += 64) {  // attn_tile_sum_k (:447-459), tile sums added in order
      int n = std::min(64, seq - start);
      float s[256];
      for (int i = 0; i < 256; ++i) s[i] = i < n ? expf(sc[start + i] - mx) : 0.0f;
      sum += tree256(s);
    }
    for (int d = 0; d < c.v_head; ++d) {  // attn_tile_accum_k (:461-470) + attn_finish_k (:472-475)
      float o = 0;
      for (int start = 0; start < seq; start += 64) {
        int n = std::min(64, seq - start);
        float acc = 0;
        for (int t = 0; t < n; ++t) {
          float p = bf(expf(sc[start + t] - mx) / sum);
          acc = fmaf(p, Vb[(size_t)(start + t) * VD + h * c.v_head + d], acc);
        }
        o += acc;
      }
      out[h * c.v_head + d] = bf16_bits(o);
    }
  }
}

// micro-tiles per span of the kx attention schedule: a function of the sequence length only
int ox_mla_span_tiles(int seq) {
  int tiles = (seq + 63) / 64, st = 1;
  while (tiles > 64 * st) st *= 2;
  return st;
}

// absorbed attention in the kx schedule over the latent cache of one sequence.
// cache bf16 [seq][kv_rank + qk_rope]; qabs f32 [heads][kv_rank + qk_rope] (bf16 values):
// W_UK^T q_nope then rotated q_rope.  out: o_lat bf16 [heads][kv_rank].
static void attn_kx_seq(const ox_config &c, const uint16_t *cache, int seq, const float *qabs, uint16_t *o_lat) {
  const int R = c.kv_rank, KVA = c.kv_rank + c.qk_rope;
  float rs, ms;
  ox_softmax_scale(&c, &rs, &ms);
  const int tiles = (seq + 63) / 64, st = ox_mla_span_tiles(seq), spans = (tiles + st - 1) / st;
#pragma omp parallel for schedule(static)
  for (int h = 0; h < c.heads; ++h) {
    const float *q = qabs + (size_t)h * KVA;
    std::vector<float> pm(spans), pz(spans), po((size_t)spans * R);
    for (int sp = 0; sp < spans; ++sp) {
      float M = -INFINITY, Z = 0.0f;
      std::vector<float> O(R, 0.0f);
      for (int tile = sp * st; tile < std::min(tiles, (sp + 1) * st); ++tile) {
        const int t0 = tile * 64, n = std::min(64, seq - t0);
        float s[64], p[64];
        float mt = -INFINITY;
        for (int l = 0; l < 64; ++l) {
          if (l < n) {
            const uint16_t *row = cache + (size_t)(t0 + l) * KVA;
            float acc = 0.0f;
            for (int i = 0; i < KVA; ++i) acc = fmaf(bf16_val(row[i]), q[i], acc);
            s[l] = bf(bf(acc) * rs * ms * ms);
          } else {
            s[l] = -INFINITY;
          }
          mt = fmaxf(mt, s[l]);
        }
        const float Mn = fmaxf(M, mt);
        const float alpha = exp_kx(M - Mn);
        for (int l = 0; l < 64; ++l) p[l] = l < n ? exp_kx(s[l] - Mn) : 0.0f;
        float pp[64];
        memcpy(pp, p, sizeof pp);
        const float zt = butterfly(pp, 64);
        Z = fmaf(Z, alpha, zt);
        for (int i = 0; i < R; ++i) {
          float o = O[i] * alpha;
          for (int l = 0; l < n; ++l) o = fmaf(bf(p[l]), bf16_val(cache[(size_t)(t0 + l) * KVA + i]), o);
          O[i] = o;
        }
        M = Mn;
      }
      pm[sp] = M; pz[sp] = Z;
      memcpy(&po[(size_t)sp * R], O.data(), sizeof(float) * R);
    }
    float M = -INFINITY;
    for (int sp = 0; sp < spans; ++sp) M = fmaxf(M, pm[sp]);
    float Z = 0.0f;
    std::vector<float> O(R, 0.0f);
    for (int sp = 0; sp < spans; ++sp) {
      const float w = exp_kx(pm[sp] - M);
      Z = fmaf(pz[sp], w, Z);
      for (int i = 0; i < R; ++i) O[i] = fmaf(po[(size_t)sp * R + i], w, O[i]);
    }
    for (int i = 0; i < R; ++i) o_lat[(size_t)h * R + i] = bf16_bits(O[i] / Z);
  }
}
// the same attention with the reference's three passes and rounding points (:414-475) applied to the
// absorbed operands: s = bf(bf(q.k)*scale); m = max; Z = sum expf(s-m); p = bf(expf(s-m)/Z); o = bf(sum p*c)
static void attn_ref_absorbed_seq(const ox_config &c, const uint16_t *cache, int seq, const float *qabs, uint16_t *o_lat) {
  const int R = c.kv_rank, KVA = c.kv_rank + c.qk_rope;
  float rs, ms;
  ox_softmax_scale(&c, &rs, &ms);
#pragma omp parallel for schedule(static)
  for (int h = 0; h < c.heads; ++h) {
    const float *q = qabs + (size_t)h * KVA;
    std::vector<float> s(seq);
    float m = -INFINITY;
    for (int t = 0; t < seq; ++t) {
      float acc = 0.0f;
      for (int i = 0; i < KVA; ++i) acc = fmaf(bf16_val(cache[(size_t)t * KVA + i]), q[i], acc);
      s[t] = bf(bf(acc) * rs * ms * ms);
      m = fmaxf(m, s[t]);
    }
    float Z = 0.0f;
    for (int t = 0; t < seq; ++t) Z += expf(s[t] - m);
    std::vector<float> O(R, 0.0f);
    for (int t = 0; t < seq; ++t) {
      const float p = bf(expf(s[t] - m) / Z);
      for (int i = 0; i < R; ++i) O[i] = fmaf(p, bf16_val(cache[(size_t)t * KVA + i]), O[i]);
    }
    for (int i = 0; i < R; ++i) o_lat[(size_t)h * R + i] = bf16_bits(O[i]);
  }
}
// BASELINE config 3 as an operator: cache bf16, sequence b at cache + b*seq_stride; qabs f32
// [batch][heads][kv_rank+qk_rope]; o_lat bf16 [batch][heads][kv_rank]
void ox_mla_decode(const ox_config *c, const uint16_t *cache, size_t seq_stride, const float *qabs, uint16_t *o_lat,
                   int batch, int seq, int mode) {
  const size_t KVA = c->kv_rank + c->qk_rope;
  for (int b = 0; b < batch; ++b) {
    const uint16_t *cb = cache + (size_t)b * seq_stride;
    const float *qb = qabs + (size_t)b * c->heads * KVA;
    uint16_t *ob = o_lat + (size_t)b * c->heads * c->kv_rank;
    if (mode) attn_kx_seq(*c, cb, seq, qb, ob);
    else attn_ref_absorbed_seq(*c, cb, seq, qb, ob);
  }
}
static void attn_kx(const ox_model *m, const OxLayer &L, int b, int seq, const float *qabs, uint16_t *o_lat) {
  const size_t KVA = m->c.kv_rank + m->c.qk_rope;
  attn_kx_seq(m->c, &L.latent[(size_t)b * m->c.max_context * KVA], seq, qabs, o_lat);
}

// one decode step of every sequence in the batch at position pos (:801-884); returns sampled ids if sample
static void model_step(ox_model *m, const uint32_t *ids, int B, int pos, int sample, uint32_t *out_ids) {
  const ox_config &c = m->c;
  const int H = c.hidden, QK = c.qk_nope + c.qk_rope, KD = c.heads * QK, VD = c.heads * c.v_head;
  const int KVA = c.kv_rank + c.qk_rope, R = c.kv_rank, mode = m->mode;
  const uint16_t *tab = &m->rope_tab[(size_t)pos * c.qk_rope];
  std::vector<uint16_t> n(H), qa(c.q_rank), q(KD), kva(KVA), att(VD), o(H), tmp;
  for (int b = 0; b < B; ++b) {
    uint16_t *x = &m->x[(size_t)b * H];
    memcpy(x, &m->embed[(size_t)ids[b] * H], (size_t)H * 2);  // embed_token (:651-655)
    for (int l = 0; l < c.n_layers; ++l) {
      OxLayer &L = m->layers[l];
      rmsnorm_row(x, L.input_ln.data(), n.data(), H, c.rms_eps, mode);                       // :812
      mv(m, L.qa, n.data(), qa.data(), c.q_rank, H);                                          // :813
      { std::vector<uint16_t> t(qa); rmsnorm_row(t.data(), L.qa_ln.data(), qa.data(), c.q_rank, c.rms_eps, mode); }  // :814
      mv(m, L.qb, qa.data(), q.data(), KD, c.q_rank);                                         // :815
      mv(m, L.kva, n.data(), kva.data(), KVA, H);                                             // :816
      { std::vector<uint16_t> t(kva.begin(), kva.begin() + R);
        rmsnorm_row(t.data(), L.kv_ln.data(), kva.data(), R, c.rms_eps, mode); }              // :817 (first kv_rank only)
      // RoPE on the shared k_rope and on every head's q_rope (:346-357)
      std::vector<float> kr_in(c.qk_rope), kr(c.qk_rope), qf(KD), q_rot(KD);
      for (int i = 0; i < c.qk_rope; ++i) kr_in[i] = bf16_val(kva[R + i]);
      rope_apply(kr_in.data(), kr.data(), tab, c.qk_rope);
      for (int i = 0; i < KD; ++i) qf[i] = bf16_val(q[i]);
      q_rot = qf;
      for (int h = 0; h < c.heads; ++h) rope_apply(&qf[h * QK + c.qk_nope], &q_rot[h * QK + c.qk_nope], tab, c.qk_rope);
      // latent cache row (both modes keep it; identical information to the reference's K/V)
      uint16_t *lat = &L.latent[((size_t)b * c.max_context + pos) * KVA];
      memcpy(lat, kva.data(), (size_t)R * 2);
      for (int i = 0; i < c.qk_rope; ++i) lat[R + i] = bf16_bits(kr[i]);
      if (!mode) {
        // kv_b projection, split into K nope and V, K rope broadcast to every head (:818-820), stored as fp32 (:824)
        std::vector<uint16_t> kv((size_t)c.heads * (c.qk_nope + c.v_head));
        mv(m, L.kvb, kva.data(), kv.data(), c.heads * (c.qk_nope + c.v_head), R);
        float *Kp = &L.K[((size_t)b * c.max_context + pos) * KD], *Vp = &L.V[((size_t)b * c.max_context + pos) * VD];
        for (int h = 0; h < c.heads; ++h) {
          for (int d = 0; d < c.qk_nope; ++d) Kp[h * QK + d] = bf16_val(kv[(size_t)h * (c.qk_nope + c.v_head) + d]);
          for (int d = 0; d < c.qk_rope; ++d) Kp[h * QK + c.qk_nope + d] = kr[d];
          for (int d = 0; d < c.v_head; ++d) Vp[h * c.v_head + d] = bf16_val(kv[(size_t)h * (c.qk_nope + c.v_head) + c.qk_nope + d]);
        }
        attn_ref(m, L, b, pos + 1, q_rot.data(), att.data());                                 // :825
      } else {
        // absorbed: q_lat[h][c] = bf(sum_d W_UK[h][d][c] q_nope[h][d]): eight chains over d = j, j+8, ...
        // then ((0+1)+(2+3))+((4+5)+(6+7))
        std::vector<float> qabs((size_t)c.heads * KVA);
#pragma omp parallel for schedule(static)
        for (int h = 0; h < c.heads; ++h) {
          for (int cc = 0; cc < R; ++cc) {
            float ch[8];
            for (int j = 0; j < 8; ++j) {
              float acc = 0.0f;
              for (int d = j; d < c.qk_nope; d += 8)
                acc = fmaf(bf16_val(L.kvb[((size_t)h * (c.qk_nope + c.v_head) + d) * R + cc]), qf[h * QK + d], acc);
              ch[j] = acc;
            }
            qabs[(size_t)h * KVA + cc] = bf(((ch[0] + ch[1]) + (ch[2] + ch[3])) + ((ch[4] + ch[5]) + (ch[6] + ch[7])));
          }
          for (int i = 0; i < c.qk_rope; ++i) qabs[(size_t)h * KVA + R + i] = q_rot[h * QK + c.qk_nope + i];
        }
        std::vector<uint16_t> o_lat((size_t)c.heads * R);
        attn_kx(m, L, b, pos + 1, qabs.data(), o_lat.data());
        // o[h] = bf(W_UV[h] o_lat[h])
        for (int h = 0; h < c.heads; ++h)
          ox_gemv_bf16(&L.kvb[((size_t)h * (c.qk_nope + c.v_head) + c.qk_nope) * R], &o_lat[(size_t)h * R],
                       &att[(size_t)h * c.v_head], c.v_head, R, 1, 0, 1);
      }
      mv(m, L.o, att.data(), o.data(), H, VD);                                                // :826
      for (int i = 0; i < H; ++i) x[i] = bf16_bits(bf16_val(x[i]) + bf16_val(o[i]));           // :827
      rmsnorm_row(x, L.post_ln.data(), n.data(), H, c.rms_eps, mode);                         // :829
      if (l < c.first_dense) {  // bf16_mlp (:674-686) on down = 0
        const int D = c.dense_inter;
        std::vector<uint16_t> g(D), u(D), mid(D), y(H);
        mv(m, L.dgate, n.data(), g.data(), D, H);
        mv(m, L.dup, n.data(), u.data(), D, H);
        for (int r = 0; r < D; ++r) mid[r] = bf16_bits(swiglu_m(bf16_val(g[r]), bf16_val(u[r]), mode));
        mv(m, L.ddown, mid.data(), y.data(), H, D);
        for (int i = 0; i < H; ++i) {
          float down = bf(0.0f + bf16_val(y[i]));                                             // :684
          x[i] = bf16_bits(bf16_val(x[i]) + down);                                            // :877
        }
      } else {
        ox_moe_weights w = {L.router.data(), L.router_bias.data(), L.gate_p.data(), L.gate_s.data(), L.up_p.data(),
                            L.up_s.data(), L.down_p.data(), L.down_s.data(), L.sh_gate.data(), L.sh_up.data(),
                            L.sh_down.data()};
        ExpertSource source = [m, l](int e) {
          const OxLayer::Expert &x = expert_on_demand(m, l, e);
          return ExpertView{x.gate_p.data(), x.gate_s.data(), x.up_p.data(), x.up_s.data(), x.down_p.data(),
                            x.down_s.data()};
        };
        moe_layer_impl(&w, n.data(), x, 1, H, c.moe_inter, c.shared_inter, c.experts, c.topk, c.routed_scale, 0, mode,
                       nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, m->on_demand ? &source : nullptr);
      }
    }
    if (sample) {  // final norm, lm_head, lowest-index argmax over bf16-rounded logits (:880-881, :718-734)
      rmsnorm_row(x, m->final_norm.data(), n.data(), H, c.rms_eps, mode);
      std::vector<uint16_t> lg(c.vocab);
      mv(m, m->lm_head, n.data(), lg.data(), c.vocab, H);
      float best = -INFINITY;
      uint32_t tok = 0;
      for (int v = 0; v < c.vocab; ++v) {
        float f = bf16_val(lg[v]);
        m->last_logits[(size_t)b * c.vocab + v] = f;
        if (f > best) best = f, tok = (uint32_t)v;
      }
      out_ids[b] = tok;
    }
  }
}

// generate(): prefill token by token, sampling only on the last prompt token, then decode (:885-890).
// prompt u32 [B][P]; out u32 [B][n_tokens]; counts i32 [B] = ids emitted (generation stops before EOS
// unless ignore_eos).  Returns 0, or 1 on a bad argument.
int ox_generate(ox_model *m, const uint32_t *prompt, int B, int P, int n_tokens, int ignore_eos, uint32_t *out,
                int *counts) {
  const ox_config &c = m->c;
  if (B < 1 || B > c.max_batch || P < 1 || n_tokens < 1 || P + n_tokens > c.max_context) return 1;
  for (int i = 0; i < B * P; ++i)
    if (prompt[i] >= (uint32_t)c.vocab) return 1;
  std::vector<uint32_t> cur(B), next(B);
  for (int i = 0; i < P; ++i) {
    for (int b = 0; b < B; ++b) cur[b] = prompt[(size_t)b * P + i];
    model_step(m, cur.data(), B, i, i + 1 == P, next.data());
  }
  std::vector<int> done(B, 0);
  for (int b = 0; b < B; ++b) counts[b] = 0;
  for (int i = 0; i < n_tokens; ++i) {
    for (int b = 0; b < B; ++b) {
      if (!done[b] && !ignore_eos && next[b] == c.eos_id) done[b] = 1;
      if (!done[b]) out[(size_t)b * n_tokens + counts[b]++] = next[b];
    }
    if (i + 1 < n_tokens) {
      cur = next;
      model_step(m, cur.data(), B, P + i, 1, next.data());
    }
  }
  return 0;
}
// One step of run() (:801-884) for every sequence of the batch at position pos, so that a caller can walk a long
// generation itself (and watch it).  ids u32 [B]; out_ids u32 [B] is written when sample is set.  Returns 0, or 1 on
// a bad argument.
int ox_model_step(ox_model *m, const uint32_t *ids, int B, int pos, int sample, uint32_t *out_ids) {
  const ox_config &c = m->c;
  if (B < 1 || B > c.max_batch || pos < 0 || pos >= c.max_context || (sample && !out_ids)) return 1;
  for (int b = 0; b < B; ++b)
    if (ids[b] >= (uint32_t)c.vocab) return 1;
  model_step(m, ids, B, pos, sample, out_ids);
  return 0;
}
const float *ox_model_logits(ox_model *m) { return m->last_logits.data(); }
const uint16_t *ox_model_hidden(ox_model *m) { return m->x.data(); }
const uint16_t *ox_model_latent(ox_model *m, int layer) { return m->layers[layer].latent.data(); }

void ox_moe_layer(const ox_moe_weights *w, const uint16_t *n, uint16_t *x, int tokens, int hidden, int moe_inter,
                  int shared_inter, int experts, int topk, float routed_scale, uint32_t flags, int mode,
                  float *o_logits, uint16_t *o_ids, float *o_weights, uint16_t *o_mid, uint16_t *o_eout) {
  moe_layer_impl(w, n, x, tokens, hidden, moe_inter, shared_inter, experts, topk, routed_scale, flags, mode, o_logits,
                 o_ids, o_weights, o_mid, o_eout, nullptr, nullptr);
}
// the same layer with the expert ids u16 [T, topk] and routing weights f32 [T, topk] given
void ox_moe_layer_routed(const ox_moe_weights *w, const uint16_t *n, uint16_t *x, int tokens, int hidden, int moe_inter,
                         int shared_inter, int experts, int topk, uint32_t flags, int mode, const uint16_t *ids,
                         const float *weights) {
  moe_layer_impl(w, n, x, tokens, hidden, moe_inter, shared_inter, experts, topk, 0.0f, flags, mode, nullptr, nullptr,
                 nullptr, nullptr, nullptr, ids, weights);
}

int ox_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
void ox_set_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}

}  // extern "C"
