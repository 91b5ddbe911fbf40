// kx_cli.cpp -- the executor boundary of the reference, on top of the C ABI.
//
// Reference: main(), args(), token_ids() and the JSON line of src/kimi_exec.cu
// (:532-557, :895-904); its caller blok/runtime.py:70-95 passes
//   --index <file> --prompt-tokens <id,id,...> --tokens <n>
// reads one JSON line {"status":"ok","token_ids":[...]} from stdout and treats a
// non-zero exit code as failure, surfacing stderr.  The same contract holds
// here.  With --index the weights are read from the checkpoint the index describes
// (runtime_index() + validate_forward_contract(), :559-585, :736-778): the stack's shapes are taken
// from the index and --layers truncates it (the full 61 layers do not fit one GPU's HBM).  Without
// --index the weights are seeded random-init.  --layers / --seed / --topk / --ignore-eos / --yarn-factor /
// --prefill-chunk / --print-config are additions.
//
// Constants.  A checkpoint run (--index) uses the reference's constants (:176-186), in particular its YaRN
// factor 64 (:184), so that the same checkpoint gives the reference's arithmetic; a seeded random-init run keeps
// the library default of 32 (the synthetic benchmark configurations).  --yarn-factor overrides either.
// Truncation.  A checkpoint with more layers than fit one GPU is never truncated silently: without --layers such a
// run is an error that says so; with --layers the JSON line also carries "layers_run" and "layers_in_checkpoint".
#include <errno.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <string>
#include <vector>
#include "../../include/kx.h"

[[noreturn]] static void die(const std::string &m) {  // :495-498
  fprintf(stderr, "%s\n", m.c_str());
  exit(1);
}
static uint64_t u64(const char *s, const char *what) {  // :504-510
  char *end = nullptr;
  errno = 0;
  unsigned long long v = strtoull(s, &end, 10);
  if (errno || end == s || *end) die(std::string("bad ") + what);
  return v;
}

int main(int argc, char **argv) {
  std::string prompt_tokens, index;
  uint64_t tokens = 0, layers = 0, seed = 0, topk = 0, prefill_chunk = 1;
  int ignore_eos = 0, print_config = 0;
  double yarn_factor = 0.0;
  for (int i = 1; i < argc; i += 2) {
    std::string f = argv[i];
    if (f == "--ignore-eos") { ignore_eos = 1; --i; continue; }
    if (f == "--print-config") { print_config = 1; --i; continue; }
    if (i + 1 >= argc) die("usage: kx-kimi-exec [--index runtime-index.blok] --prompt-tokens ids --tokens n [--layers n] [--seed n] [--topk n] [--yarn-factor f] [--prefill-chunk n] [--ignore-eos] [--print-config]");
    if (f == "--index") index = argv[i + 1];
    else if (f == "--prompt-tokens") prompt_tokens = argv[i + 1];
    else if (f == "--tokens") tokens = u64(argv[i + 1], "tokens");
    else if (f == "--layers") layers = u64(argv[i + 1], "layers");
    else if (f == "--seed") seed = u64(argv[i + 1], "seed");
    else if (f == "--topk") topk = u64(argv[i + 1], "topk");
    else if (f == "--yarn-factor") {
      char *end = nullptr;
      yarn_factor = strtod(argv[i + 1], &end);
      if (end == argv[i + 1] || *end || !(yarn_factor >= 1.0)) die("bad yarn factor");
    }
    else if (f == "--prefill-chunk") prefill_chunk = u64(argv[i + 1], "prefill chunk");  // not in the reference: prompt positions per prefill step
    else die("unknown flag: " + f);  // :540
  }
  if (prompt_tokens.empty() || tokens == 0) die("bad args");  // :542
  kx_config cfg;
  if (kx_config_default(&cfg)) die(kx_last_error());
  if (topk) cfg.topk = (int32_t)topk;
  if (!index.empty() && kx_index_infer_config(index.c_str(), &cfg)) die(kx_last_error());
  if (!index.empty()) cfg.yarn_factor = 64.0f;  // YARN_FACTOR (:184); the other constants of :176-186 are the defaults
  if (yarn_factor > 0.0) cfg.yarn_factor = (float)yarn_factor;
  const int32_t checkpoint_layers = index.empty() ? 0 : cfg.n_layers;
  std::vector<uint32_t> ids;  // token_ids(), :546-557
  size_t at = 0;
  while (at <= prompt_tokens.size()) {
    size_t comma = prompt_tokens.find(',', at);
    std::string v = prompt_tokens.substr(at, comma == std::string::npos ? std::string::npos : comma - at);
    uint64_t id = u64(v.c_str(), "prompt token");
    if (id >= (uint64_t)cfg.vocab) die("prompt token outside vocabulary");
    ids.push_back((uint32_t)id);
    if (comma == std::string::npos) break;
    at = comma + 1;
  }
  if (ids.empty()) die("prompt token list is empty");
  if (layers > 61) die("bad layers");
  if (layers == 0) {
    if (index.empty()) {
      layers = 24;  // the truncation of the benchmark configurations: 24 Kimi-K2 layers fill one GPU
    } else {
      uint64_t weights = 0, cache = 0, scratch = 0;
      cfg.max_batch = 1;
      cfg.max_context = 4096;
      if (kx_model_bytes(&cfg, &weights, &cache, &scratch)) die(kx_last_error());
      if (weights > 280ull * 1000 * 1000 * 1000)  // more than one MI355X holds
        die("the checkpoint has " + std::to_string(cfg.n_layers) + " layers (" + std::to_string(weights / 1000000000ull) +
            " GB): they do not fit one GPU; pass --layers n to run the first n layers only (the result is then not the full model's)");
      layers = (uint64_t)cfg.n_layers;
    }
  }
  if (!index.empty() && layers > (uint64_t)cfg.n_layers) die("the checkpoint has fewer layers than --layers");
  const uint64_t max_context = 262144;  // :180
  if (tokens > max_context || ids.size() > max_context - tokens) die("requested sequence exceeds Kimi context");  // :784
  cfg.n_layers = (int32_t)layers;
  cfg.seed = seed;
  cfg.max_batch = 1;
  cfg.max_context = (int32_t)(ids.size() + tokens);
  if (prefill_chunk < 1 || prefill_chunk > 2048) die("bad prefill chunk: 1 to 2048 positions per step");
  if (print_config) {  // what the run would use, without touching a GPU
    printf("{\"n_layers\":%d,\"layers_in_checkpoint\":%d,\"first_dense\":%d,\"hidden\":%d,\"heads\":%d,\"q_rank\":%d,\"kv_rank\":%d,"
           "\"qk_nope\":%d,\"qk_rope\":%d,\"v_head\":%d,\"experts\":%d,\"topk\":%d,\"moe_inter\":%d,\"shared_inter\":%d,"
           "\"dense_inter\":%d,\"vocab\":%d,\"max_context\":%d,\"eos_id\":%u,\"rms_eps\":%.9g,\"rope_theta\":%.9g,"
           "\"routed_scale\":%.9g,\"yarn_factor\":%.9g,\"yarn_beta_fast\":%.9g,\"yarn_beta_slow\":%.9g,\"yarn_orig_ctx\":%.9g,"
           "\"yarn_mscale_all_dim\":%.9g,\"prefill_chunk\":%llu}\n",
           cfg.n_layers, checkpoint_layers, cfg.first_dense, cfg.hidden, cfg.heads, cfg.q_rank, cfg.kv_rank, cfg.qk_nope, cfg.qk_rope,
           cfg.v_head, cfg.experts, cfg.topk, cfg.moe_inter, cfg.shared_inter, cfg.dense_inter, cfg.vocab, cfg.max_context, cfg.eos_id,
           cfg.rms_eps, cfg.rope_theta, cfg.routed_scale, cfg.yarn_factor, cfg.yarn_beta_fast, cfg.yarn_beta_slow, cfg.yarn_orig_ctx,
           cfg.yarn_mscale_all_dim, (unsigned long long)prefill_chunk);
    return 0;
  }
  kx_model *m = nullptr;
  if (index.empty() ? kx_model_create(&cfg, &m) : kx_model_load(&cfg, index.c_str(), &m)) die(kx_last_error());
  if (prefill_chunk != 1 && kx_model_set_prefill_chunk(m, (int32_t)prefill_chunk)) {
    std::string msg = kx_last_error();
    kx_model_destroy(m);
    die(msg);
  }
  std::vector<uint32_t> out(tokens);
  int32_t count = 0;
  if (kx_generate(m, ids.data(), 1, (int32_t)ids.size(), (int32_t)tokens, ignore_eos, out.data(), &count)) {
    std::string msg = kx_last_error();
    kx_model_destroy(m);
    die(msg);
  }
  kx_model_destroy(m);
  printf("{\"status\":\"ok\",\"token_ids\":[");  // :901-903
  for (int i = 0; i < count; ++i) printf("%s%u", i ? "," : "", out[i]);
  if (checkpoint_layers > cfg.n_layers) printf("],\"layers_run\":%d,\"layers_in_checkpoint\":%d}\n", cfg.n_layers, checkpoint_layers);
  else printf("]}\n");
  return 0;
}
