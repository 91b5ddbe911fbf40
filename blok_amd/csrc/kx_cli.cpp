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
// --index the weights are seeded random-init.  --layers / --seed / --topk / --ignore-eos are additions.
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
  int ignore_eos = 0;
  for (int i = 1; i < argc; i += 2) {
    std::string f = argv[i];
    if (f == "--ignore-eos") { ignore_eos = 1; --i; continue; }
    if (i + 1 >= argc) die("usage: kx-kimi-exec [--index runtime-index.blok] --prompt-tokens ids --tokens n [--layers n] [--seed n] [--topk n] [--prefill-chunk n] [--ignore-eos]");
    if (f == "--index") index = argv[i + 1];
    else if (f == "--prompt-tokens") prompt_tokens = argv[i + 1];
    else if (f == "--tokens") tokens = u64(argv[i + 1], "tokens");
    else if (f == "--layers") layers = u64(argv[i + 1], "layers");
    else if (f == "--seed") seed = u64(argv[i + 1], "seed");
    else if (f == "--topk") topk = u64(argv[i + 1], "topk");
    else if (f == "--prefill-chunk") prefill_chunk = u64(argv[i + 1], "prefill chunk");  // not in the reference: prompt positions per prefill step
    else die("unknown flag: " + f);  // :540
  }
  if (prompt_tokens.empty() || tokens == 0) die("bad args");  // :542
  kx_config cfg;
  if (kx_config_default(&cfg)) die(kx_last_error());
  if (topk) cfg.topk = (int32_t)topk;
  if (!index.empty() && kx_index_infer_config(index.c_str(), &cfg)) die(kx_last_error());
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
  if (layers == 0) layers = index.empty() || cfg.n_layers > 24 ? 24 : (uint64_t)cfg.n_layers;  // 24 Kimi-K2 layers fill one GPU
  if (!index.empty() && layers > (uint64_t)cfg.n_layers) die("the checkpoint has fewer layers than --layers");
  const uint64_t max_context = 262144;  // :180
  if (tokens > max_context || ids.size() > max_context - tokens) die("requested sequence exceeds Kimi context");  // :784
  cfg.n_layers = (int32_t)layers;
  cfg.seed = seed;
  cfg.max_batch = 1;
  cfg.max_context = (int32_t)(ids.size() + tokens);
  kx_model *m = nullptr;
  if (index.empty() ? kx_model_create(&cfg, &m) : kx_model_load(&cfg, index.c_str(), &m)) die(kx_last_error());
  if (prefill_chunk != 1 && kx_model_set_prefill_chunk(m, prefill_chunk > 1000 ? 1000 : (int32_t)prefill_chunk)) {
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
  printf("]}\n");
  return 0;
}
