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
// No function of the hot path is pinned by a golden vector of the reference:
// the reference holds none for arithmetic (its only test, scripts/test_host.py,
// pins the argv/JSON boundary).
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <algorithm>
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

void ox_fill_normal_bf16(uint16_t *out, uint64_t n, uint64_t seed, uint64_t tid, float sigma, int absval) {
  uint64_t key = rng_key(seed, tid);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) {
    uint16_t h = bf16_bits(rng_normal_f32(key, (uint64_t)i, sigma));
    out[i] = absval ? (uint16_t)(h & 0x7fff) : h;
  }
}
void ox_fill_normal_f32(float *out, uint64_t n, uint64_t seed, uint64_t tid, float sigma) {
  uint64_t key = rng_key(seed, tid);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) out[i] = rng_normal_f32(key, (uint64_t)i, sigma);
}
void ox_fill_words_u32(uint32_t *out, uint64_t n, uint64_t seed, uint64_t tid) {
  uint64_t key = rng_key(seed, tid);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i)
    out[i] = (uint32_t)(rng_u64(key, (uint64_t)i >> 1) >> (32u * (uint32_t)(i & 1)));
}

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
                  float *o_logits, uint16_t *o_ids, float *o_weights, uint16_t *o_mid, uint16_t *o_eout) {
  const int H = hidden, I = moe_inter, SI = shared_inter, E = experts, K = topk;
  std::vector<float> logits((size_t)tokens * E), weights((size_t)tokens * K);
  std::vector<uint16_t> ids((size_t)tokens * K);
  ox_gemv_bf16(w->router_gate, n, logits.data(), E, H, tokens, 1, mode);  // :838
  ox_router_topk(logits.data(), w->router_bias, ids.data(), weights.data(), tokens, E, K, routed_scale, mode);
  if (o_logits) memcpy(o_logits, logits.data(), logits.size() * 4);
  if (o_ids) memcpy(o_ids, ids.data(), ids.size() * 2);
  if (o_weights) memcpy(o_weights, weights.data(), weights.size() * 4);
  std::vector<uint16_t> g(I), u(I), mid(I), y(H), sg(SI), su(SI), smid(SI), sy(H);
  for (int t = 0; t < tokens; ++t) {
    const uint16_t *nt = n + (size_t)t * H;
    std::vector<float> down(H, 0.0f);
    for (int slot = 0; slot < K; ++slot) {  // :845-870
      int e = ids[(size_t)t * K + slot];
      size_t wo = (size_t)e * I * (H / 8), so = (size_t)e * I * (H / 32);
      ox_i4_gemv(w->gate_packed + wo, w->gate_scale + so, nt, g.data(), I, H, 1, mode);
      ox_i4_gemv(w->up_packed + wo, w->up_scale + so, nt, u.data(), I, H, 1, mode);
      for (int r = 0; r < I; ++r) mid[r] = bf16_bits(swiglu_m(bf16_val(g[r]), bf16_val(u[r]), mode));
      size_t dwo = (size_t)e * H * (I / 8), dso = (size_t)e * H * (I / 32);
      ox_i4_gemv(w->down_packed + dwo, w->down_scale + dso, mid.data(), y.data(), H, I, 1, mode);
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
