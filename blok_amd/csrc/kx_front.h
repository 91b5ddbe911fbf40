// kx_front.h -- launch interface of the fused front of the attention block (kx_front.hip).
#pragma once
#include <hip/hip_runtime.h>
#include "kx_attn_parts.h"
#include "kx_dense.h"

// words of the `hand` array for a model: the tagged q_a, kv_a and q values of one token
inline size_t kx_front_hand_words(int q_rank, int kva, int q_rows) { return (size_t)q_rank + kva + q_rows; }
int kx_attn_front_launch(const KxGemvArgs &g_qkv, const KxGemvArgs &g_qb, const QAbsArgs &q, uint32_t *hand, uint32_t tag, int *err,
                         bool *done, hipStream_t st);
int kx_attn_back_launch(const KxGemvArgs &g_uv, const KxGemvArgs &g_o, uint32_t *hand, uint32_t tag, int *err, bool *done, hipStream_t st);
