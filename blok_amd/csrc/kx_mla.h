// kx_mla.h -- internal launch interface of the attention kernels (kx_mla.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include "../../include/kx.h"

// 64-position tiles per span of the attention schedule; depends on the sequence length only
int kx_mla_span_tiles(int seq);
// floats of partial results (m, z, o) the attention needs for `batch` sequences up to max_seq
size_t kx_mla_partial_floats(int batch, int heads, int kv_rank, int max_seq);

// seqs > 0 (a prefill step): token i * seqs + b is position pos + i of sequence b; rope_row points at the table row of
// position pos and the rows of the following positions lie behind it.
// q absorb + rope(q); when cache != nullptr one extra block per token also finishes kv_a
// (RMSNorm of the latent, rope of the shared key) and writes the cache row of position pos
int kx_q_absorb_launch(const uint16_t *q, const uint16_t *kvb, const uint16_t *rope_row, float *qabs, int tokens,
                       int heads, int nope, int rope, int v_head, int kv_rank, const uint16_t *kva, int kva_stride,
                       const uint16_t *w_kv_ln, uint16_t *cache, size_t seq_stride, int pos, float eps, hipStream_t st,
                       int seqs = 0);
struct KxMlaPartials {
  const float *pm, *pz, *po;  // [batch][spans][heads], same, [batch][spans][heads][kv_rank]
  int spans;
};
// seqs > 0 (a prefill step): the `batch` entries are positions x sequences, entry i * seqs + b = position i of
// sequence b, which reads cache block b and attends seq - (batch / seqs - 1) + i positions (the last position: seq).
// scores + online softmax + PV per span; the merge is left to the caller (kx_mla_combine_launch, or the W_UV GEMV
// when there are at most 64 spans)
int kx_mla_partials_launch(const kx_config *c, const uint16_t *cache, size_t seq_stride, const float *qabs, float *partial,
                           int batch, int seq, KxMlaPartials *out, hipStream_t st, int seqs = 0, int kernel = KX_MLA_AUTO);
// the merge of the span partials as a kernel of its own: o_lat bf16 [batch][heads][kv_rank] (any number of spans)
int kx_mla_combine_launch(const KxMlaPartials &p, uint16_t *o_lat, int batch, int heads, hipStream_t st);
int kx_mla_attend_launch(const kx_config *c, const uint16_t *cache, size_t seq_stride, const float *qabs, float *partial,
                         uint16_t *o_lat, int batch, int seq, hipStream_t st, int seqs = 0, int kernel = KX_MLA_AUTO);
