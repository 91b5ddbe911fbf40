// kx_dense.h -- internal launch interface of the bf16 GEMV family (kx_dense.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

enum {
  KX_EPI_BF16 = 0,        // y = bf(sum)                           matvec_bf16_k
  KX_EPI_F32 = 1,         // y = sum (router logits)               matvec_bf16_f32_k
  KX_EPI_SWIGLU = 2,      // two matrices: bf(bf(silu(bf(g)))*bf(u)) silu_mul_k
  KX_EPI_RESID = 3,       // x = bf(x + bf(sum))                   add_k
  KX_EPI_MOE_COMBINE = 4, // shared down + routed combine + residual
  KX_EPI_ARGMAX = 5       // bf16-rounded logits as f32 for the argmax reduction
};


struct KxGemvArgs {
  const uint16_t *w0;  // bf16 [rows, cols]
  const uint16_t *w1;  // second matrix for KX_EPI_SWIGLU
  const uint16_t *x;   // bf16 activations, row stride x_stride
  int x_stride;
  void *out;
  int out_stride;
  int rows, cols, tokens;
  int nw, rs, nt, epi;  // set by kx_gemv_launch
  // optional block structure (absorbed W_UV: one 128-row block per head inside kv_b):
  // output rows [k*row_block, (k+1)*row_block) use weight rows k*w_block_stride + w_block_off + r
  // and the activation row at x + k*x_block_stride.  row_block == 0: plain matrix.
  int row_block, w_block_stride, w_block_off, x_block_stride;
  // optional prologue: x is RMS-normed with these weights before use (at most 4 tokens);
  // norm_out, if set, receives the normed rows [tokens][cols]
  const uint16_t *norm_w;
  float norm_eps;
  uint16_t *norm_out;
  // optional: x[t] of block (head) k is the merge of attention partials, bf(O/Z), instead of a.x
  const float *mla_pm, *mla_pz, *mla_po;
  int mla_spans, mla_heads;
  // KX_EPI_MOE_COMBINE
  const uint16_t *expert_out;  // bf16 [tokens*topk, rows]
  const float *route_w;        // f32 [tokens, topk]
  int topk;
  uint32_t flags;              // bit 0: MOE_COMBINE overwrites x; KX_GEMV_COHERENT_OUT: see below
};
// F32 and BF16 epilogues: store the outputs with device-scope stores (another workgroup of the launch reads them)
#define KX_GEMV_COHERENT_OUT 2u

int kx_gemv_launch(int epi, KxGemvArgs a, hipStream_t st);
// The q_b GEMV (g: rows = heads * (nope + rope), bf16 epilogue) that also finishes the query: the workgroup that
// completes a head last computes q_abs of that head (W_UK absorb + RoPE, the sums of q_absorb_k), and one extra
// workgroup norms kv_a, rotates the rope key and writes the cache row.  head_count: one zeroed int per head.
// Returns KX_OK with *fused = false, having launched nothing, when the shapes do not allow it.
struct QAbsArgs;
int kx_gemv_absorb_launch(KxGemvArgs g, const QAbsArgs &q, bool *fused, hipStream_t st);
int kx_rmsnorm_launch(const uint16_t *x, const uint16_t *w, uint16_t *y, int tokens, int n, int x_stride,
                      int y_stride, float eps, hipStream_t st);
int kx_argmax_launch(const float *logits, int tokens, int n, int stride, uint32_t *out, float *scratch, hipStream_t st);
#define KX_ARGMAX_SCRATCH_FLOATS(tokens) ((size_t)(tokens) * 128)

// kx_i4.hip
// What the routed down launch needs to finish the MoE layer itself (up to 4 tokens): its workgroups and those of the
// shared expert's down GEMV, which ride in the same launch, count themselves in per block of output rows; whichever
// completes a block combines it (expert_accum_k / round_bf16_k :399-407, the shared add :684, the residual :877).
struct KxMoeTail {
  int *counter;          // one per row block, zero between launches; nullptr: no tail
  const int *n_active;   // experts with work (device value written by the routing)
  int shared_chunks;     // chunks of the shared down GEMV per row block
  const uint16_t *sy;    // bf16 [tokens, rows]: the shared down GEMV's output (device-scope stores)
  const float *route_w;  // f32 [tokens, topk]
  uint16_t *x;           // residual rows, updated in place
  int x_stride, tokens, topk;
  uint32_t flags;        // bit 0: x = down instead of x += down
};
// The routed down GEMV over the work list + the shared expert's down GEMV (shared: weights, activations, rows, cols,
// tokens; its output goes to tail.sy) + the combine, in one launch.  Returns KX_OK with *fused = false, having
// launched nothing, when the shapes do not allow it.
int kx_i4_down_shared_launch(const uint32_t *packed, const uint16_t *scale, const uint16_t *x, uint16_t *out, const int4 *work,
                             const int *pairs, int rows, int cols, int x_div, size_t expert_words, size_t expert_scales,
                             int n_slots, KxGemvArgs shared, KxMoeTail tail, bool *fused, hipStream_t st);
// The same with the routed gate/up + SwiGLU in front, as one resident launch whose workgroups hand the mid values to
// each other as tagged words (kx_hand.h; hand: n_slots * inter words, tag in [1, 65535] and different from the last
// launch's, err: the flag a wait that gives up sets).  *fused = false, nothing launched, when shapes or device do not fit.
int kx_i4_routed_shared_launch(const uint32_t *gate_packed, const uint16_t *gate_scale, const uint32_t *up_packed, const uint16_t *up_scale,
                               const uint32_t *down_packed, const uint16_t *down_scale, const uint16_t *x, uint16_t *mid, uint16_t *eout,
                               const int4 *work, const int *pairs, int hidden, int inter, int topk, int n_slots, KxGemvArgs shared,
                               KxMoeTail tail, uint32_t *hand, uint32_t tag, int *err, bool *fused, hipStream_t st);
// the launch shape kx_gemv_launch would give a GEMV (fills a.nw, a.rs, a.nt, a.epi); returns rows per chunk or -1
int kx_gemv_plan(int epi, KxGemvArgs &a, int *ri);
// cnt_lo..cnt_hi: only the experts of the work list with that many pairs are processed (0, INT_MAX: all)
int kx_i4_launch(bool dual, const uint32_t *packed0, const uint16_t *scale0, const uint32_t *packed1,
                 const uint16_t *scale1, const uint16_t *x, uint16_t *out, const int4 *work,
                 const int *pairs, int n_pairs, int rows,
                 int cols, int x_div, size_t expert_words, size_t expert_scales, int tt, int n_slots,
                 int cnt_lo, int cnt_hi, hipStream_t st, int chunk_mult = 1);

// kx_router.hip
int kx_router_topk_launch(const float *logits, const float *bias, uint16_t *ids, float *weights, int tokens,
                          int experts, int topk, float routed_scale, hipStream_t st);
int kx_gemv_pair_route_launch(KxGemvArgs shared_gate_up, KxGemvArgs router, const float *bias, uint16_t *ids, float *weights,
                              int experts, int topk, float routed_scale, int *counts, int *offsets, int *pairs, int4 *work,
                              int *n_active, int *counter, bool *fused, hipStream_t st, int4 *pair_work = nullptr);
// The router's logits GEMV (fp32 epilogue) of any number of tokens.  From 8 to 32 tokens the launch also does the
// routing -- *routed = true; counters: 1 + ceil(tokens / 4) ints, zero before the call and left at zero --, otherwise
// kx_route_launch follows.
int kx_gemv_route_launch(KxGemvArgs router, const float *bias, uint16_t *ids, float *weights, int experts, int topk,
                         float routed_scale, int *counts, int *offsets, int *pairs, int4 *work, int *n_active, int *counters,
                         bool *routed, hipStream_t st, int4 *pair_work = nullptr);
int kx_route_launch(const float *logits, const float *bias, uint16_t *ids, float *weights, int tokens, int experts,
                    int topk, float routed_scale, int *counts, int *offsets, int *pairs, int4 *work, int *n_active,
                    hipStream_t st, int4 *pair_work = nullptr);
int kx_bucket_launch(const uint16_t *ids, int tokens, int experts, int topk, int *counts, int *offsets,
                     int *pairs, int4 *work, int *n_active, hipStream_t st, int4 *pair_work = nullptr);

// kx_prefill.hip
// outputs of the grouped GEMM: bf16; fp32 unrounded; fp32 holding the bf16-rounded value; bf16 residual add into out
enum { KX_GG_BF16 = 0, KX_GG_F32 = 1, KX_GG_F32_OF_BF16 = 2, KX_GG_RESID = 3 };
int kx_grouped_gemm_launch(bool dual, bool i4, const void *w0, const uint16_t *s0, const void *w1, const uint16_t *s1,
                           const uint16_t *x, void *out, int out_mode, const int4 *work, const int *pairs, int n_pairs,
                           int n_slots, int N, int K, int x_div, size_t expert_w, size_t expert_s, int n_pairs_max,
                           hipStream_t st, int cnt_lo = 0);
// kx_i4mm.hip: the experts of the work list with cnt_lo .. cnt_hi pairs as W4A16 products on the matrix cores with the
// weights streamed into registers, up to 32 tokens of an expert per pass (passes: grid depth; an expert's pairs beyond
// 32 * passes are not computed).  out[pair][N] = W[expert] x[pair / x_div], or swiglu(W0 x, W1 x) with two matrices.
// *done = false (nothing launched) when the shape is not the kernel's.
int kx_i4mm_launch(bool dual, const uint32_t *w0, const uint16_t *s0, const uint32_t *w1, const uint16_t *s1, const uint16_t *x,
                   uint16_t *out, const int4 *work, const int *pairs, int n_slots, int N, int K, int x_div, size_t expert_w,
                   size_t expert_s, int cnt_lo, int cnt_hi, int passes, bool *done, hipStream_t st);
// kx_skinny.hip: one tile of up to 32 tokens against a bf16 matrix (two for SwiGLU) on the matrix cores, out_mode as
// above.  *done = false (nothing launched) when the shape is not the kernel's.
int kx_skinny_gemm_launch(bool dual, const uint16_t *w0, const uint16_t *w1, const uint16_t *x, int x_stride, void *out,
                          int out_stride, int out_mode, int tokens, int rows, int cols, bool *done, hipStream_t st);
int kx_moe_combine_launch(const uint16_t *eout, const float *rw, const uint16_t *sy, uint16_t *x, int tokens, int hidden,
                          int topk, uint32_t flags, hipStream_t st);

// kx_moe.hip: the decode layer with the post-attention RMSNorm fused into the router GEMV.
// When norm_w is set, d_x is normed on the fly and the normed rows are written to d_n first.
struct kx_moe_workspace;
// flag for kx_moe_layer_launch (beside bit 0): keep the shared down GEMV and the combine a launch of their own
#define KX_MOE_SEPARATE_TAIL 0x100u
// 5 to 32 tokens: the shared expert's GEMVs on the matrix cores (kx_skinny.hip; tolerance instead of bit parity)
#define KX_MOE_SHARED_MATRIX_CORES 0x200u
// 5 tokens and more: the routed experts with three or more pairs as W4A16 grouped GEMMs on the matrix cores
// (kx_prefill.hip) instead of the GEMV kernels: such an expert's weights are streamed and dequantised once for all its
// tokens (tolerance instead of bit parity); the experts with one or two pairs keep the GEMV kernel.  From 32 to 64
// tokens: the experts with two or more pairs through kx_i4mm.hip (weights dequantized in registers, f16 products)
#define KX_MOE_ROUTED_MATRIX_CORES 0x400u
// internal (not among the public flags): the layer's first launch -- normed row in d_n, router logits, routing, shared
// gate/up -- has been done by the caller's own launch (kx_front.hip's back launch with kx_moe_head_args): one token
#define KX_MOE_HEAD_DONE 0x800u
// internal: one token, the routed experts (gate/up, down, shared down, combine) as one resident launch where shapes
// and device allow it; the workspace must have been given an error flag (kx_moe_workspace_set_err)
#define KX_MOE_ROUTED_RESIDENT 0x1000u
void kx_moe_workspace_set_err(kx_moe_workspace *ws, int *d_err);
int *kx_moe_workspace_n_active(kx_moe_workspace *ws);  // device address of the count of distinct experts of the last call
// the flags a caller of kx_moe_decode_layer may pass (include/kx.h documents them)
#define KX_MOE_PUBLIC_FLAGS (1u | KX_MOE_SEPARATE_TAIL | KX_MOE_SHARED_MATRIX_CORES | KX_MOE_ROUTED_MATRIX_CORES)
int kx_moe_layer_launch(const kx_config *c, const kx_moe_weights *w, kx_moe_workspace *ws, void *d_n, void *d_x,
                        int tokens, uint32_t flags, const uint16_t *norm_w, hipStream_t st, bool timed);
