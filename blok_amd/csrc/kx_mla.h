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

int kx_kv_finish_launch(const uint16_t *qkv, const uint16_t *w_qa_ln, const uint16_t *w_kv_ln, const uint16_t *rope_row,
                        uint16_t *qa_out, uint16_t *cache, int tokens, int q_rank, int kv_rank, int rope,
                        size_t seq_stride, int pos, float eps, hipStream_t st);
int kx_q_absorb_launch(const uint16_t *q, const uint16_t *kvb, const uint16_t *rope_row, float *qabs, int tokens,
                       int heads, int nope, int rope, int v_head, int kv_rank, hipStream_t st);
int kx_mla_attend_launch(const kx_config *c, const uint16_t *cache, size_t seq_stride, const float *qabs, float *partial,
                         uint16_t *o_lat, int batch, int seq, hipStream_t st);
