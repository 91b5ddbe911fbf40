// kx_load.h -- copies checkpoint tensors from their files into the resident arena.
//
// Reference: load_tensor() / load_tensor_slice_into() (src/kimi_exec.cu:608-649) read the
// 4096-aligned extent [off, off+bytes) of a tensor through uGDS into a fresh device buffer and
// skip data-off bytes, once per use inside the layer loop.  Here every tensor is read once, at
// load time: reader threads pread the aligned extents piece by piece into pinned staging
// buffers (O_DIRECT where the file system takes it) and copy the data range to its place in HBM.
#pragma once
#include <vector>
#include "kx_index.h"

struct KxLoadItem {
  const KxTensorRec *t;
  char *dst;   // device address of the first data byte
  bool widen;  // bf16 in the file, f32 in HBM
};

// bytes: data bytes copied; seconds: wall time of the whole copy
int kx_load_run(const std::vector<KxLoadItem> &items, uint64_t *bytes, double *seconds);
