// Host-side code under AddressSanitizer + UndefinedBehaviorSanitizer (no GPU): the checkpoint index parser and the
// tokenizer of the library (blok_amd/csrc/kx_index.hip, kx_tok.hip: host-only files that parse untrusted input,
// compiled here as plain C++) and the CPU oracle (oracle/kx_oracle.cpp).  The test that builds this program
// (tests/test_sanitizers.py) hands it a directory of inputs, valid and malformed; every call must come back with a
// status, and the sanitizers must have nothing to report.  The reference has no sanitizer build
// (CMakeLists.txt:14-16 only turns warnings into errors).
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <string>
#include <vector>
#include "../include/kx.h"

// what kx_util.hip provides inside the library
static thread_local char g_err[512] = "";
void kx_set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
}
extern "C" const char *kx_last_error(void) { return g_err; }
extern "C" int kx_config_default(kx_config *c) {
  memset(c, 0, sizeof *c);
  c->n_layers = 3; c->first_dense = 1; c->hidden = 1024; c->heads = 8; c->qk_nope = 128; c->qk_rope = 64; c->v_head = 128;
  c->q_rank = 512; c->kv_rank = 512; c->experts = 16; c->topk = 4; c->moe_inter = 1024; c->shared_inter = 512;
  c->dense_inter = 1536; c->vocab = 2048; c->max_batch = 1; c->max_context = 16; c->eos_id = 2047;
  c->rms_eps = 1e-5f; c->rope_theta = 50000.0f; c->routed_scale = 2.827f; c->yarn_factor = 32.0f; c->yarn_beta_fast = 32.0f;
  c->yarn_beta_slow = 1.0f; c->yarn_orig_ctx = 4096.0f; c->yarn_mscale_all_dim = 1.0f; c->init_sigma = 0.02f;
  c->expert_scale_sigma = 0.02f; c->seed = 1234;
  return 0;
}

// oracle entry points used below (oracle/kx_oracle.cpp)
extern "C" {
struct ox_model;
ox_model *ox_model_create(const kx_config *cfg, int mode);
void ox_model_destroy(ox_model *m);
int ox_generate(ox_model *m, const uint32_t *prompt, int B, int P, int n_tokens, int ignore_eos, uint32_t *out, int *counts);
void ox_i4_gemv(const uint32_t *packed, const uint16_t *scale, const uint16_t *x, uint16_t *y, int rows, int cols, int tokens, int mode);
void ox_fill_words_u32(uint32_t *out, uint64_t n, uint64_t seed, uint64_t tid);
void ox_fill_normal_bf16(uint16_t *out, uint64_t n, uint64_t seed, uint64_t tid, float sigma, int absval);
int ox_bucket(const uint16_t *ids, int tokens, int experts, int topk, int *counts, int *offsets, int *pairs, int *active);
}

static int failures = 0;
#define EXPECT(cond, what)                                   \
  do {                                                       \
    if (!(cond)) {                                           \
      fprintf(stderr, "FAILED: %s (%s)\n", what, g_err);     \
      ++failures;                                            \
    }                                                        \
  } while (0)

int main(int argc, char **argv) {
  if (argc != 2) return 64;
  const std::string dir = argv[1];
  kx_config cfg;
  kx_config_default(&cfg);

  // ---- index parser: the good index, then every malformed one the test wrote (bad_*.blok) ----
  uint64_t n = 0, bytes = 0;
  EXPECT(kx_index_check(&cfg, (dir + "/good/runtime-index.blok").c_str(), &n, &bytes) == 0 && n > 0, "good index");
  kx_config got = cfg;
  EXPECT(kx_index_infer_config((dir + "/good/runtime-index.blok").c_str(), &got) == 0 && got.hidden == cfg.hidden, "infer config");
  for (int i = 0;; ++i) {
    const std::string p = dir + "/bad_" + std::to_string(i) + ".blok";
    FILE *f = fopen(p.c_str(), "rb");
    if (!f) break;
    fclose(f);
    EXPECT(kx_index_check(&cfg, p.c_str(), &n, &bytes) != 0, p.c_str());
    kx_config scratch = cfg;
    (void)kx_index_infer_config(p.c_str(), &scratch);  // any status; it must not crash
  }
  EXPECT(kx_index_check(&cfg, (dir + "/nowhere/runtime-index.blok").c_str(), &n, &bytes) != 0, "missing index");

  // ---- tokenizer: a good file, malformed files (tok_bad_*.blok), awkward strings ----
  kx_tokenizer *tk = nullptr;
  EXPECT(kx_tokenizer_open((dir + "/tokenizer.blok").c_str(), &tk) == 0 && tk, "good tokenizer");
  for (int i = 0;; ++i) {
    const std::string p = dir + "/tok_bad_" + std::to_string(i) + ".blok";
    FILE *f = fopen(p.c_str(), "rb");
    if (!f) break;
    fclose(f);
    kx_tokenizer *bad = nullptr;
    EXPECT(kx_tokenizer_open(p.c_str(), &bad) != 0 && !bad, p.c_str());
  }
  if (tk) {
    FILE *f = fopen((dir + "/strings.bin").c_str(), "rb");  // length-prefixed byte strings, some of them invalid UTF-8
    EXPECT(f != nullptr, "strings.bin");
    uint32_t len = 0;
    while (f && fread(&len, 4, 1, f) == 1) {
      std::string s(len, '\0');
      if (len && fread(&s[0], 1, len, f) != len) break;
      std::vector<uint32_t> ends(len + 1), ids(len + 64);
      size_t ne = 0, ni = 0;
      EXPECT(kx_pretokenize(s.data(), s.size(), ends.data(), ends.size(), &ne) == 0 && (ne == 0 || ends[ne - 1] == len), "pretokenize");
      for (int special = 0; special < 2; ++special) {
        EXPECT(kx_tokenizer_encode(tk, s.data(), s.size(), special, ids.data(), ids.size(), &ni) == 0, "encode");
        std::string back(len + 1, '\0');
        size_t nb = 0;
        EXPECT(kx_tokenizer_decode(tk, ids.data(), ni, &back[0], back.size(), &nb) == 0 && nb == len && memcmp(back.data(), s.data(), len) == 0,
               "decode(encode) is the identity");
      }
      EXPECT(kx_encode_prompt(tk, s.data(), s.size(), ids.data(), 2, &ni) != 0 || ni <= 2, "a buffer that is too small is an error");
      uint32_t wild[3] = {0xffffffffu, 1u << 30, 5};
      char out[8];
      size_t no = 0;
      (void)kx_tokenizer_decode(tk, wild, 3, out, sizeof out, &no);  // unknown ids: an error, not a crash
    }
    if (f) fclose(f);
    kx_tokenizer_close(tk);
  }

  // ---- oracle: a few steps of the small stack in both schedules, a ragged GEMV, the bucketing ----
  for (int mode = 0; mode < 2; ++mode) {
    ox_model *m = ox_model_create(&cfg, mode);
    uint32_t prompt[3] = {5, 2047, 0}, out[2] = {0, 0};
    int counts = 0;
    EXPECT(ox_generate(m, prompt, 1, 3, 2, 1, out, &counts) == 0 && counts == 2 && out[0] < 2048 && out[1] < 2048, "oracle generate");
    EXPECT(ox_generate(m, prompt, 1, 3, 64, 1, out, &counts) == 1, "oracle rejects a sequence beyond the context");
    ox_model_destroy(m);
    std::vector<uint32_t> w(64 * 1024 / 8);
    std::vector<uint16_t> sc(64 * 1024 / 32), x(3 * 1024), y(3 * 64);
    ox_fill_words_u32(w.data(), w.size(), 1, 1);
    ox_fill_normal_bf16(sc.data(), sc.size(), 1, 2, 0.02f, 1);
    ox_fill_normal_bf16(x.data(), x.size(), 1, 3, 1.0f, 0);
    ox_i4_gemv(w.data(), sc.data(), x.data(), y.data(), 64, 1024, 3, mode);
  }
  {
    const int T = 37, E = 16, K = 4;
    std::vector<uint16_t> ids(T * K);
    for (int i = 0; i < T * K; ++i) ids[i] = (uint16_t)((i * 7 + i / K) % E);
    std::vector<int> counts(E), offsets(E + 1), pairs(T * K), active(E);
    const int na = ox_bucket(ids.data(), T, E, K, counts.data(), offsets.data(), pairs.data(), active.data());
    EXPECT(na > 0 && na <= E && offsets[E] == T * K, "oracle bucket");
  }
  printf("sanitize driver: %d failure(s)\n", failures);
  return failures ? 1 : 0;
}
