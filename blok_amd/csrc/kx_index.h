// kx_index.h -- the checkpoint side of the boundary: runtime-index.blok.
//
// Reference: the index is written by scripts/model_fetch.py materialize()
// (:116-131, one `tensor` line of 14 fields per checkpoint tensor) and read by
// runtime_index() (src/kimi_exec.cu:559-585); validate_forward_contract()
// (:736-778) fixes which (layer, role, slot, expert) keys a forward pass needs
// and their dtype / shape / byte count.
#pragma once
#include <stdint.h>
#include <string>
#include <unordered_map>
#include <vector>
#include "kx_common.h"

struct KxTensorRec {  // one `tensor` line (struct Tensor, src/kimi_exec.cu:27-31)
  std::string name, role, slot, dtype, shape, file;
  uint64_t off = 0, bytes = 0, align = 4096, data = 0, data_bytes = 0;
  int layer = -1, expert = -1;
};

struct KxIndex {
  std::string path;
  std::unordered_map<std::string, KxTensorRec> tensors;  // key "layer:expert:role:slot" (:579)
  const KxTensorRec *find(int layer, const char *role, const char *slot, int expert = -1) const;
};

// where a checkpoint tensor lives in the resident model
enum KxSlot {
  KXS_EMBED, KXS_FINAL_NORM, KXS_LM_HEAD,
  KXS_INPUT_LN, KXS_QA, KXS_QA_LN, KXS_QB, KXS_KVA, KXS_KV_LN, KXS_KVB, KXS_O, KXS_POST_LN,
  KXS_DENSE_GATE, KXS_DENSE_UP, KXS_DENSE_DOWN,
  KXS_ROUTER, KXS_ROUTER_BIAS,
  KXS_GATE_P, KXS_GATE_S, KXS_UP_P, KXS_UP_S, KXS_DOWN_P, KXS_DOWN_S,
  KXS_SH_GATE, KXS_SH_UP, KXS_SH_DOWN
};

struct KxNeed {  // one tensor the forward pass of `cfg` reads
  const KxTensorRec *t;
  KxSlot slot;
  int layer, expert;
};

// Parses the index.  Errors carry the reference's messages (:561-583).
int kx_index_parse(const char *path, KxIndex &out);
// The forward contract for the first cfg->n_layers layers with cfg's shapes; fills `needs` in a fixed order.
int kx_index_contract(const KxIndex &ix, const kx_config *cfg, std::vector<KxNeed> &needs);
