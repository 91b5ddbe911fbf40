// kx_index.hip -- runtime-index.blok: parse, forward contract, shape inference (host code only).
//
// Reference: runtime_index() (src/kimi_exec.cu:559-585), need() / bf16() / validate_i4_pair()
// (:587-606) and validate_forward_contract() (:736-778).  The reference checks against the
// compile-time Kimi-K2 constants (:176-181) and wants all 61 layers; here the shapes and the
// number of layers come from a kx_config, so a truncated stack loads from the full checkpoint
// and a small test checkpoint goes through the same code.
#include <errno.h>
#include <stdlib.h>
#include <string.h>
#include "kx_index.h"

namespace {

bool parse_u64(const std::string &s, uint64_t &v) {
  if (s.empty() || s[0] == '-' || s[0] == '+') return false;
  char *end = nullptr;
  errno = 0;
  unsigned long long r = strtoull(s.c_str(), &end, 10);
  if (errno || end == s.c_str() || *end) return false;
  v = r;
  return true;
}
bool parse_int(const std::string &s, int &v) {
  char *end = nullptr;
  errno = 0;
  long r = strtol(s.c_str(), &end, 10);
  if (errno || end == s.c_str() || *end || r < INT32_MIN || r > INT32_MAX) return false;
  v = (int)r;
  return true;
}

std::string key_of(int layer, int expert, const char *role, const char *slot) {
  return std::to_string(layer) + ":" + std::to_string(expert) + ":" + role + ":" + slot;
}

// whitespace-separated fields of one line
void split_fields(const std::string &line, std::vector<std::string> &out) {
  out.clear();
  size_t i = 0;
  const size_t n = line.size();
  while (i < n) {
    while (i < n && (line[i] == ' ' || line[i] == '\t' || line[i] == '\r')) ++i;
    size_t b = i;
    while (i < n && line[i] != ' ' && line[i] != '\t' && line[i] != '\r') ++i;
    if (i > b) out.emplace_back(line, b, i - b);
  }
}

std::string shape_text(uint64_t rows, uint64_t cols) {
  return cols ? std::to_string(rows) + "x" + std::to_string(cols) : std::to_string(rows);
}

struct Contract {
  const KxIndex &ix;
  std::vector<KxNeed> &needs;
  // a tensor of `dtype` with the given shape (cols == 0: one dimension); element size from the dtype
  int want(int layer, const char *role, const char *slot, int expert, const char *dtype, uint64_t rows, uint64_t cols,
           KxSlot where, const char *what) {
    const KxTensorRec *t = ix.find(layer, role, slot, expert);
    KX_REQUIRE(t, "missing runtime tensor: %s", key_of(layer, expert, role, slot).c_str());  // :590
    const uint64_t esz = strcmp(dtype, "bf16") == 0 ? 2 : 4;
    const uint64_t bytes = rows * (cols ? cols : 1) * esz;
    KX_REQUIRE(t->dtype == dtype && t->shape == shape_text(rows, cols) && t->data_bytes == bytes,
               "%s: %s (%s %s, %llu bytes; expected %s %s, %llu bytes)", what, t->name.c_str(), t->dtype.c_str(),
               t->shape.c_str(), (unsigned long long)t->data_bytes, dtype, shape_text(rows, cols).c_str(),
               (unsigned long long)bytes);  // :598, :600-605, :764
    needs.push_back(KxNeed{t, where, layer, expert});
    return KX_OK;
  }
  int bf16(int layer, const char *role, const char *slot, uint64_t rows, uint64_t cols, KxSlot where) {
    return want(layer, role, slot, -1, "bf16", rows, cols, where, "bad bf16 tensor contract");
  }
  int i4_pair(int layer, int expert, const char *proj, uint64_t rows, uint64_t cols, KxSlot wp, KxSlot ws) {  // :599-606
    const std::string p = std::string(proj) + ".weight_packed", s = std::string(proj) + ".weight_scale";
    int rc = want(layer, "routed_expert", p.c_str(), expert, "i32", rows, cols / 8, wp, "bad routed expert packed shape");
    if (rc) return rc;
    return want(layer, "routed_expert", s.c_str(), expert, "bf16", rows, cols / 32, ws, "bad routed expert scale shape");
  }
};

}  // namespace

const KxTensorRec *KxIndex::find(int layer, const char *role, const char *slot, int expert) const {
  auto it = tensors.find(key_of(layer, expert, role, slot));
  return it == tensors.end() ? nullptr : &it->second;
}

int kx_index_parse(const char *path, KxIndex &out) {
  KX_REQUIRE(path && path[0], "kx_index: empty index path");
  FILE *f = fopen(path, "rb");
  KX_REQUIRE(f, "missing runtime-index.blok: %s (%s)", path, strerror(errno));  // :561
  out.path = path;
  out.tensors.clear();
  std::string dir = path;
  const size_t slash = dir.find_last_of('/');
  dir = slash == std::string::npos ? std::string(".") : dir.substr(0, slash);
  std::string line;
  std::vector<std::string> fld;
  char *buf = nullptr;
  size_t cap = 0;
  long lineno = 0;
  int rc = KX_OK;
  auto fail = [&](const char *msg, const std::string &arg) {
    kx_set_error("%s%s%s (%s:%ld)", msg, arg.empty() ? "" : ": ", arg.c_str(), path, lineno);
    rc = KX_ERR_ARG;
  };
  ssize_t got;
  while (!rc && (got = getline(&buf, &cap, f)) >= 0) {
    ++lineno;
    while (got > 0 && (buf[got - 1] == '\n' || buf[got - 1] == '\r')) --got;
    line.assign(buf, (size_t)got);
    if (lineno == 1) {
      if (line != "blok-runtime-index-v1") fail("bad runtime index header", "");  // :565
      continue;
    }
    if (line.compare(0, 7, "tensor ") != 0) { fail("bad runtime index line", ""); break; }  // :567
    split_fields(line, fld);
    if (fld.size() < 14) { fail("incomplete runtime tensor line", ""); break; }             // :571-572
    if (fld.size() > 14) { fail("runtime tensor path cannot contain whitespace", ""); break; }  // :573-574
    KxTensorRec t;
    t.name = fld[1]; t.role = fld[2]; t.slot = fld[5]; t.dtype = fld[6]; t.shape = fld[7]; t.file = fld[13];
    if (!parse_int(fld[3], t.layer)) { fail("bad layer", fld[3]); break; }    // :575
    if (!parse_int(fld[4], t.expert)) { fail("bad expert", fld[4]); break; }  // :576
    if (!parse_u64(fld[8], t.off) || !parse_u64(fld[9], t.bytes) || !parse_u64(fld[10], t.align) ||
        !parse_u64(fld[11], t.data) || !parse_u64(fld[12], t.data_bytes)) { fail("incomplete runtime tensor line", ""); break; }
    if (t.file[0] != '/') t.file = dir + "/" + t.file;  // an index that moves with its shards
    const std::string key = key_of(t.layer, t.expert, t.role.c_str(), t.slot.c_str());
    if (!out.tensors.emplace(key, std::move(t)).second) { fail("duplicate runtime tensor key", key); break; }  // :580
  }
  free(buf);
  fclose(f);
  if (rc) return rc;
  KX_REQUIRE(lineno >= 1, "bad runtime index header (%s is empty)", path);
  KX_REQUIRE(!out.tensors.empty(), "runtime index has no file-backed tensors (%s)", path);  // :583
  return KX_OK;
}

int kx_index_contract(const KxIndex &ix, const kx_config *c, std::vector<KxNeed> &needs) {
  needs.clear();
  for (const auto &kv : ix.tensors) {  // :737-745
    const KxTensorRec &t = kv.second;
    KX_REQUIRE(!t.slot.empty() && !t.dtype.empty() && !t.shape.empty(), "runtime index has incomplete tensor metadata: %s", t.name.c_str());
    KX_REQUIRE(t.layer >= -1 && t.expert >= -1 && t.expert < c->experts, "runtime index has out-of-range Kimi coordinates: %s", t.name.c_str());
    KX_REQUIRE(t.off <= UINT64_MAX - t.bytes && t.data <= UINT64_MAX - t.data_bytes, "runtime index has invalid tensor extent: %s", t.name.c_str());
    KX_REQUIRE(t.align == 4096 && t.off % t.align == 0 && t.bytes % t.align == 0 && t.data >= t.off &&
                   t.data_bytes <= t.bytes && t.data - t.off <= t.bytes - t.data_bytes,
               "runtime index has invalid tensor extent: %s", t.name.c_str());
  }
  const uint64_t H = c->hidden, V = c->vocab, I = c->moe_inter, SI = c->shared_inter, D = c->dense_inter;
  const uint64_t KD = (uint64_t)c->heads * (c->qk_nope + c->qk_rope), VD = (uint64_t)c->heads * c->v_head;
  const uint64_t KVA = c->kv_rank + c->qk_rope, KVB = (uint64_t)c->heads * (c->qk_nope + c->v_head);
  Contract k{ix, needs};
  int rc;
#define KX_TRY(call) do { if ((rc = (call))) return rc; } while (0)
  KX_TRY(k.bf16(-1, "resident", "embed_tokens", V, H, KXS_EMBED));  // :775-777
  KX_TRY(k.bf16(-1, "resident", "norm", H, 0, KXS_FINAL_NORM));
  KX_TRY(k.bf16(-1, "resident", "lm_head", V, H, KXS_LM_HEAD));
  for (int l = 0; l < c->n_layers; ++l) {
    const char *att = "attention_resident";
    KX_TRY(k.bf16(l, att, "q_a_proj", c->q_rank, H, KXS_QA));  // :747-755
    KX_TRY(k.bf16(l, att, "q_a_layernorm", c->q_rank, 0, KXS_QA_LN));
    KX_TRY(k.bf16(l, att, "q_b_proj", KD, c->q_rank, KXS_QB));
    KX_TRY(k.bf16(l, att, "kv_a_proj_with_mqa", KVA, H, KXS_KVA));
    KX_TRY(k.bf16(l, att, "kv_a_layernorm", c->kv_rank, 0, KXS_KV_LN));
    KX_TRY(k.bf16(l, att, "kv_b_proj", KVB, c->kv_rank, KXS_KVB));
    KX_TRY(k.bf16(l, att, "o_proj", H, VD, KXS_O));
    KX_TRY(k.bf16(l, "resident", "input_layernorm", H, 0, KXS_INPUT_LN));
    KX_TRY(k.bf16(l, "resident", "post_attention_layernorm", H, 0, KXS_POST_LN));
    if (l < c->first_dense) {  // :756-761
      KX_TRY(k.bf16(l, "dense_ffn_rowcol", "gate_proj", D, H, KXS_DENSE_GATE));
      KX_TRY(k.bf16(l, "dense_ffn_rowcol", "up_proj", D, H, KXS_DENSE_UP));
      KX_TRY(k.bf16(l, "dense_ffn_rowcol", "down_proj", H, D, KXS_DENSE_DOWN));
      continue;
    }
    KX_TRY(k.bf16(l, "router", "gate", c->experts, H, KXS_ROUTER));  // :762
    KX_TRY(k.want(l, "router", "e_score_correction_bias", -1, "bf16", c->experts, 0, KXS_ROUTER_BIAS, "bad router correction bias"));
    KX_TRY(k.bf16(l, "shared_expert_resident", "gate_proj", SI, H, KXS_SH_GATE));  // :767-769
    KX_TRY(k.bf16(l, "shared_expert_resident", "up_proj", SI, H, KXS_SH_UP));
    KX_TRY(k.bf16(l, "shared_expert_resident", "down_proj", H, SI, KXS_SH_DOWN));
    for (int e = 0; e < c->experts; ++e) {  // :770-774
      KX_TRY(k.i4_pair(l, e, "gate_proj", I, H, KXS_GATE_P, KXS_GATE_S));
      KX_TRY(k.i4_pair(l, e, "up_proj", I, H, KXS_UP_P, KXS_UP_S));
      KX_TRY(k.i4_pair(l, e, "down_proj", H, I, KXS_DOWN_P, KXS_DOWN_S));
    }
  }
#undef KX_TRY
  return KX_OK;
}

// ---- C ABI ---------------------------------------------------------------------------------
static int kx_index_check_body(const kx_config *cfg, const char *index_path, uint64_t *n_tensors, uint64_t *weight_bytes) {
  KX_REQUIRE(cfg, "kx_index_check: null config");
  KxIndex ix;
  int rc = kx_index_parse(index_path, ix);
  if (rc) return rc;
  std::vector<KxNeed> needs;
  if ((rc = kx_index_contract(ix, cfg, needs))) return rc;
  uint64_t bytes = 0;
  for (const KxNeed &n : needs) bytes += n.t->data_bytes;
  if (n_tensors) *n_tensors = needs.size();
  if (weight_bytes) *weight_bytes = bytes;
  return KX_OK;
}

// Shapes of the checkpoint an index describes, written over the matching fields of *cfg.
static int kx_index_infer_config_body(const char *index_path, kx_config *cfg) {
  KX_REQUIRE(cfg, "kx_index_infer_config: null config");
  KxIndex ix;
  int rc = kx_index_parse(index_path, ix);
  if (rc) return rc;
  auto dims = [&](const KxTensorRec *t, uint64_t &r, uint64_t &c2) {
    const size_t x = t->shape.find('x');
    c2 = 0;
    if (x == std::string::npos) return parse_u64(t->shape, r);
    return parse_u64(t->shape.substr(0, x), r) && parse_u64(t->shape.substr(x + 1), c2);
  };
  uint64_t r = 0, c2 = 0;
  const KxTensorRec *t = ix.find(-1, "resident", "embed_tokens");
  KX_REQUIRE(t && dims(t, r, c2) && c2, "missing runtime tensor: %s", key_of(-1, -1, "resident", "embed_tokens").c_str());
  cfg->vocab = (int32_t)r;
  cfg->hidden = (int32_t)c2;
  int layers = 0, first_dense = 0, experts = 0;
  for (const auto &kv : ix.tensors) {
    const KxTensorRec &q = kv.second;
    if (q.layer + 1 > layers) layers = q.layer + 1;
    if (q.role == "dense_ffn_rowcol" && q.layer + 1 > first_dense) first_dense = q.layer + 1;
    if (q.role == "routed_expert" && q.expert + 1 > experts) experts = q.expert + 1;
  }
  KX_REQUIRE(layers > 0, "runtime index names no decoder layer (%s)", index_path);
  cfg->n_layers = layers;
  cfg->first_dense = first_dense;
  if ((t = ix.find(0, "attention_resident", "q_a_proj")) && dims(t, r, c2)) cfg->q_rank = (int32_t)r;
  if ((t = ix.find(0, "attention_resident", "kv_a_proj_with_mqa")) && dims(t, r, c2)) cfg->kv_rank = (int32_t)r - cfg->qk_rope;
  if ((t = ix.find(0, "attention_resident", "q_b_proj")) && dims(t, r, c2)) cfg->heads = (int32_t)(r / (uint64_t)(cfg->qk_nope + cfg->qk_rope));
  if ((t = ix.find(0, "dense_ffn_rowcol", "gate_proj")) && dims(t, r, c2)) cfg->dense_inter = (int32_t)r;
  if (first_dense < layers) {
    cfg->experts = experts;
    if (cfg->topk > experts) cfg->topk = experts;
    if ((t = ix.find(first_dense, "shared_expert_resident", "gate_proj")) && dims(t, r, c2)) cfg->shared_inter = (int32_t)r;
    if ((t = ix.find(first_dense, "routed_expert", "gate_proj.weight_scale", 0)) && dims(t, r, c2)) cfg->moe_inter = (int32_t)r;
  }
  // A checkpoint is computed with the reference's constant, YARN_FACTOR 64 (src/kimi_exec.cu:184); the library
  // default of 32 belongs to the seeded random-init configurations.  It enters the RoPE frequencies (:338) and,
  // through mscale, the softmax scale at every context length (:428-429).
  cfg->yarn_factor = 64.0f;
  return KX_OK;
}

// ---- the C ABI: every body above runs under kx_guard, so that no exception leaves the library ----
extern "C" int kx_index_check(const kx_config *cfg, const char *index_path, uint64_t *n_tensors, uint64_t *weight_bytes) {
  return kx_guard("kx_index_check", [&] { return kx_index_check_body(cfg, index_path, n_tensors, weight_bytes); });
}
extern "C" int kx_index_infer_config(const char *index_path, kx_config *cfg) {
  return kx_guard("kx_index_infer_config", [&] { return kx_index_infer_config_body(index_path, cfg); });
}
