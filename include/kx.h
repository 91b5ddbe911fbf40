/* kx.h -- C ABI of the MI355X (gfx950) implementation of blok's kimi_exec
 * forward hot path.
 *
 * The reference (akhilnairCSE110/blok) has no plugin or FFI surface: its hot
 * path is the body of one CUDA executable, src/kimi_exec.cu.  Each entry point
 * below replaces the host function or kernel of that file named in its
 * comment, with the same operand meaning; shapes default to the constants at
 * src/kimi_exec.cu:176-186.
 *
 * Conventions
 *  - every function returns 0 on success and a non-zero code on failure;
 *    kx_last_error() then returns a message (thread local).  The reference
 *    prints and exits (die(), src/kimi_exec.cu:495-498); a library cannot.
 *  - pointers named d_* are device (HBM) addresses, h_* are host addresses.
 *  - bf16 tensors are arrays of uint16_t bit patterns, row-major.
 *  - `stream` is a hipStream_t passed as void*; NULL is the default stream.
 *    Operator calls only enqueue work; they do not synchronise.
 *  - INT4 weights use the compressed-tensors pack_quantized layout the
 *    reference validates at src/kimi_exec.cu:599-606: packed int32 [N, K/8],
 *    nibble j of a word is column 8*word+j, stored value = q + 8; scales
 *    bf16 [N, K/32].
 */
#ifndef KX_H
#define KX_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* Model shape and numeric constants (src/kimi_exec.cu:176-186). */
typedef struct kx_config {
  int32_t n_layers;      /* decoder layers in the stack (reference: 61)            */
  int32_t first_dense;   /* layers [0, first_dense) use the dense MLP (reference 1) */
  int32_t hidden;        /* 7168 */
  int32_t heads;         /* 64   */
  int32_t qk_nope;       /* 128  */
  int32_t qk_rope;       /* 64   */
  int32_t v_head;        /* 128  */
  int32_t q_rank;        /* 1536 */
  int32_t kv_rank;       /* 512  */
  int32_t experts;       /* 384  */
  int32_t topk;          /* 8    */
  int32_t moe_inter;     /* 2048 */
  int32_t shared_inter;  /* 2048 */
  int32_t dense_inter;   /* 18432 */
  int32_t vocab;         /* 163840 */
  int32_t max_batch;     /* sequences decoded together                           */
  int32_t max_context;   /* positions of latent KV cache per sequence            */
  uint32_t eos_id;       /* 163586: generation stops before emitting it          */
  float rms_eps;         /* 1e-5 */
  float rope_theta;      /* 50000 */
  float routed_scale;    /* 2.827 */
  float yarn_factor;     /* 32 here; the reference pins 64 (:184)                 */
  float yarn_beta_fast;  /* 32 */
  float yarn_beta_slow;  /* 1  */
  float yarn_orig_ctx;   /* 4096 */
  float yarn_mscale_all_dim; /* 1 */
  float init_sigma;      /* std of the random-init bf16 weights (0.02)            */
  float expert_scale_sigma; /* INT4 group scales are |N(0, this)| (0.02)           */
  uint64_t seed;         /* seed of every synthetic tensor                        */
} kx_config;

/* Kimi-K2 shapes, 24 layers (1 dense + 23 MoE), batch 1, context 4096. */
int kx_config_default(kx_config *cfg);
const char *kx_last_error(void);

/* ---- device plumbing (reference: Buf / DeviceTensor, :137-174) ---------- */
int kx_device_info(char *name, size_t name_len, int32_t *compute_units, uint64_t *hbm_bytes);
int kx_dev_malloc(void **d_ptr, size_t bytes);
int kx_dev_free(void *d_ptr);
int kx_dev_memset(void *d_ptr, int value, size_t bytes, void *stream);
/* free and total device memory of the current device, in bytes (hipMemGetInfo) */
int kx_dev_mem_info(size_t *free_bytes, size_t *total_bytes);
int kx_h2d(void *d_dst, const void *h_src, size_t bytes);
int kx_d2h(void *h_dst, const void *d_src, size_t bytes);
int kx_sync(void *stream);
/* hipEvent timing on `stream` */
int kx_event_create(void **event);
int kx_event_destroy(void *event);
int kx_event_record(void *event, void *stream);
int kx_event_elapsed_ms(void *start, void *stop, float *ms); /* waits for stop */

/* Device-to-device copy by a plain kernel (16 bytes per lane); bytes and both pointers multiples of 16.
 * No counterpart in the reference: it is the known-size kernel that HBM traffic counters are scaled by. */
int kx_dev_copy(void *d_dst, const void *d_src, uint64_t bytes, void *stream);

/* ---- synthetic tensors: value = f(seed, tensor_id, index) --------------- */
int kx_fill_normal_bf16(void *d_out, uint64_t n, uint64_t seed, uint64_t tensor_id, float sigma,
                        int absval, void *stream);
int kx_fill_normal_f32(void *d_out, uint64_t n, uint64_t seed, uint64_t tensor_id, float sigma,
                       void *stream);
int kx_fill_words_u32(void *d_out, uint64_t n, uint64_t seed, uint64_t tensor_id, void *stream);
/* token ids uniform in [0, vocab): the uniform-random prompts of the benchmark configurations */
int kx_fill_tokens_u32(void *d_out, uint64_t n, uint64_t seed, uint64_t tensor_id, uint32_t vocab, void *stream);

/* ---- INT4 operators ------------------------------------------------------
 * kx_i4_unpack : nibble extraction of matvec_i4_bf16_scale_k (:309-311);
 *                d_q int8 [rows, cols] in [-8, 7].
 * kx_i4_dequant: the dequantized weight bf((float)q * scale) of :306,:312;
 *                d_w bf16 [rows, cols].
 * kx_i4_gemv   : matvec_i4_slice (:688-690) / matvec_i4_bf16_scale_k
 *                (:300-323) for T activation rows at once:
 *                y[t, r] = bf(sum_k x[t, k] * w[r, k]), x bf16 [T, cols],
 *                y bf16 [T, rows].  cols must be a multiple of 1024.         */
int kx_i4_unpack(const void *d_packed, void *d_q, int32_t rows, int32_t cols, void *stream);
int kx_i4_dequant(const void *d_packed, const void *d_scale, void *d_w, int32_t rows, int32_t cols,
                  void *stream);
int kx_i4_gemv(const void *d_packed, const void *d_scale, const void *d_x, void *d_y, int32_t rows,
               int32_t cols, int32_t tokens, void *stream);

/* ---- dense operators -----------------------------------------------------
 * kx_rmsnorm  : rmsnorm_k (:258-270); x, y bf16 [T, n], w bf16 [n].
 * kx_gemv_bf16: matvec_bf16_k (:272-284) when out_f32 == 0 (y bf16 [T, rows],
 *               rounded) and matvec_bf16_f32_k (:286-298) when out_f32 != 0
 *               (y f32 [T, rows], unrounded).  cols multiple of 512.
 * kx_lm_head_argmax: sample_lm_head (:718-734) + argmax_k (:477-493) on rows that
 *               are already normed (:880): d_logits f32 [T, vocab] receives the
 *               bf16-rounded logits bf(W n), d_ids u32 [T] the index of the
 *               largest one, the lowest index on ties, 0 when no logit compares
 *               greater than -inf.  d_scratch: T * 512 bytes.  hidden multiple of 512. */
int kx_rmsnorm(const void *d_x, const void *d_w, void *d_y, int32_t tokens, int32_t n, float eps,
               void *stream);
int kx_gemv_bf16(const void *d_w, const void *d_x, void *d_y, int32_t rows, int32_t cols,
                 int32_t tokens, int out_f32, void *stream);
int kx_lm_head_argmax(const void *d_w, const void *d_n, void *d_logits, void *d_ids, int32_t vocab,
                      int32_t hidden, int32_t tokens, void *d_scratch, void *stream);

/* kx_lm_head_argmax for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same operands and
 * results as kx_lm_head_argmax, without d_scratch: the argmax partials go to a device array that is part of
 * the library (128 KiB, held by every GPU the library runs on until the process ends), so tokens <= 256; more
 * is an error.  The call allocates nothing and frees nothing.  Every call on a GPU shares that GPU's array:
 * calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not.  Nothing in the
 * array has to be cleared between calls.  The array's address on a GPU is looked up on the first call there;
 * kx_static_scratch_init() does that look-up for the current device ahead of time (call it before a graph
 * capture begins).                                                                                        */
int kx_static_scratch_init(void);
int kx_lm_head_argmax_static(const void *d_w, const void *d_n, void *d_logits, void *d_ids, int32_t vocab,
                             int32_t hidden, int32_t tokens, void *stream);

/* ---- router --------------------------------------------------------------
 * kx_router_topk: sigmoid_k + add_bf16_k + router_topk_k (:372-397) on fp32
 *                 logits [T, E]: ids u16 [T, topk] in descending select
 *                 score, lowest index on ties; weights f32 [T, topk].
 * kx_bucket     : token -> expert bucketing (the reference's host loop at
 *                 :845 for batch 1).  counts i32 [E], offsets i32 [E+1],
 *                 pairs i32 [T*topk] holding token*topk+slot sorted by
 *                 (expert, token, slot); work i32 [E, 4] holds one record
 *                 {expert, first, last, pairs[first]} per expert with at
 *                 least one pair, in ascending expert order, followed by
 *                 {-1, 0, 0, 0} records; n_active i32 [1] counts the former. */
int kx_router_topk(const void *d_logits, const void *d_bias, void *d_ids, void *d_weights,
                   int32_t tokens, int32_t experts, int32_t topk, float routed_scale, void *stream);
int kx_bucket(const void *d_ids, int32_t tokens, int32_t experts, int32_t topk, void *d_counts,
              void *d_offsets, void *d_pairs, void *d_work, void *d_n_active, void *stream);

/* ---- one routed-MoE decode layer (the `else` branch of run(), :835-877) ---
 * Weights of one layer.  Expert tensors hold all E experts back to back.    */
typedef struct kx_moe_weights {
  const void *d_router_gate;   /* bf16 [E, hidden]                      */
  const void *d_router_bias;   /* f32  [E]                              */
  const void *d_gate_packed;   /* i32  [E, moe_inter, hidden/8]         */
  const void *d_gate_scale;    /* bf16 [E, moe_inter, hidden/32]        */
  const void *d_up_packed;     /* i32  [E, moe_inter, hidden/8]         */
  const void *d_up_scale;      /* bf16 [E, moe_inter, hidden/32]        */
  const void *d_down_packed;   /* i32  [E, hidden, moe_inter/8]         */
  const void *d_down_scale;    /* bf16 [E, hidden, moe_inter/32]        */
  const void *d_shared_gate;   /* bf16 [shared_inter, hidden]           */
  const void *d_shared_up;     /* bf16 [shared_inter, hidden]           */
  const void *d_shared_down;   /* bf16 [hidden, shared_inter]           */
} kx_moe_weights;

/* Scratch for kx_moe_decode_layer; sized for `max_tokens`. */
typedef struct kx_moe_workspace kx_moe_workspace;
int kx_moe_workspace_create(const kx_config *cfg, int32_t max_tokens, kx_moe_workspace **ws);
int kx_moe_workspace_destroy(kx_moe_workspace *ws);
/* device views of the last call's routing results (for parity checks) */
int kx_moe_workspace_views(kx_moe_workspace *ws, void **d_logits, void **d_ids, void **d_weights,
                           void **d_counts, void **d_offsets, void **d_pairs, void **d_mid,
                           void **d_expert_out);

/* d_n   bf16 [T, hidden]: the post-attention RMSNorm output (input of the FFN)
 * d_x   bf16 [T, hidden]: the residual stream; on return x = bf(x + down)
 *       with down = bf(bf(sum_slot y_slot * w_slot) + bf(shared)) (:868-877).
 * flags bit0: skip the residual add and write `down` to d_x instead.
 *       bit8: run the shared expert's down GEMV and the combine as a launch of their own even
 *             for one token (by default they ride in the routed down launch; same results).
 *       bit9: 5 to 32 tokens: the shared expert's two GEMVs as bf16 matrix-core products (another
 *             summation order: within max-rel 1e-2 of the default instead of equal to the bit).
 *       bit10: 5 tokens and more: the routed experts that have three or more (token, slot) pairs as W4A16
 *             grouped GEMMs on the matrix cores, the experts with one or two pairs through the GEMV kernel (same
 *             tolerance); from 32 to 64 tokens the experts with two or more pairs, by a kernel that dequantizes
 *             to f16 in registers.  The router is not affected by either bit, so the routing stays the default's.
 *             The decoder stack sets bit9 from 5 sequences on and bit10 from 12. */
int kx_moe_decode_layer(const kx_config *cfg, const kx_moe_weights *w, kx_moe_workspace *ws,
                        const void *d_n, void *d_x, int32_t tokens, uint32_t flags, void *stream);
/* The same layer for a prefill chunk of T tokens (BASELINE config 4): the tokens of each expert are
 * gathered into a W4A16 grouped GEMM -- INT4 words dequantized into LDS tiles of bf16 feeding
 * v_mfma_f32_32x32x16_bf16 with fp32 accumulators -- and the shared expert runs as a bf16 GEMM.
 * The reference has no batched prefill (one run() per prompt token, :886); per token the result is
 * that of kx_moe_decode_layer within max-rel 1e-2.                                               */
int kx_moe_prefill_layer(const kx_config *cfg, const kx_moe_weights *w, kx_moe_workspace *ws,
                         const void *d_n, void *d_x, int32_t tokens, uint32_t flags, void *stream);
/* per-phase kernel time of the most recent kx_moe_decode_layer_timed call, ms:
 * [0] router+bucket [1] routed gate/up [2] routed down [3] shared gate/up
 * [4] shared down + combine.  Synchronises.  The intervals are taken on `stream`: up to 4 tokens the
 * shared gate/up rides in the router's launch ([0] holds it, [3] reads about 0); with bit9 or bit10
 * the work the layer puts on its side stream lies outside [0]..[3] and is waited for inside [4].  */
int kx_moe_decode_layer_timed(const kx_config *cfg, const kx_moe_weights *w, kx_moe_workspace *ws,
                              const void *d_n, void *d_x, int32_t tokens, uint32_t flags,
                              void *stream, float *ms5);
/* One routed-expert kernel alone, on the routing that the most recent kx_moe_decode_layer call left in
 * the workspace: which = 0 gate/up + SwiGLU (:845-861), 1 down (:863-866).  For timing a kernel back
 * to back; it has no counterpart of its own in the reference.                                    */
int kx_moe_routed_only(const kx_config *cfg, const kx_moe_weights *w, kx_moe_workspace *ws,
                       const void *d_n, int32_t tokens, int32_t which, void *stream);

/* ---- MLA decode attention (tiled_attention, :692-716, on the absorbed latent cache) ----
 * kx_rope_table   : rope_k's cos/sin (:351) with the YaRN frequencies (:325-344) for positions
 *                   pos0 .. pos0+n-1; h_out bf16 [n][qk_rope]: qk_rope/2 cosines, then sines.
 * kx_softmax_scale: the two factors of the score scale (:428-429).
 * kx_q_absorb     : d_q bf16 [T][heads][qk_nope+qk_rope] (q_b output, :815) ->
 *                   d_qabs f32 [T][heads][kv_rank+qk_rope] = (bf(W_UK^T q_nope) | rope(q_rope));
 *                   d_kvb bf16 [heads*(qk_nope+v_head)][kv_rank] (kv_b_proj, :751);
 *                   d_rope_row bf16 [qk_rope] is the table row of the tokens' position.
 * kx_mla_decode   : d_cache bf16, sequence b at d_cache + b*seq_stride (elements), rows of
 *                   kv_rank+qk_rope = (normed latent | rotated rope key); attends the first
 *                   `seq` positions; d_o_lat bf16 [batch][heads][kv_rank] is the softmax-weighted
 *                   latent (W_UV is applied by the caller, kx_gemv_bf16 per head).
 *                   d_workspace: kx_mla_workspace_bytes(cfg, batch, max seq) bytes.              */
int kx_rope_table(const kx_config *cfg, int32_t pos0, int32_t n, uint16_t *h_out);
int kx_softmax_scale(const kx_config *cfg, float *rsqrt_head, float *mscale);
int kx_q_absorb(const kx_config *cfg, const void *d_q, const void *d_kvb, const void *d_rope_row,
                void *d_qabs, int32_t tokens, void *stream);
int kx_mla_workspace_bytes(const kx_config *cfg, int32_t batch, int32_t max_seq, size_t *bytes);
/* `kernel`: which kernel computes the attention partials.  KX_MLA_AUTO: the matrix-core kernel from 2048 cached
 * positions on (from 128 for five sequences and more) and the VALU kernel below; KX_MLA_VALU: the VALU kernel
 * always (fixed summation order, the one the token-identity checks rest on); KX_MLA_MATRIX_CORES: the matrix-core
 * kernel always (same values, another summation order; 64 heads).  No counterpart in the reference.        */
#define KX_MLA_AUTO 0
#define KX_MLA_VALU 1
#define KX_MLA_MATRIX_CORES 2
int kx_mla_decode(const kx_config *cfg, const void *d_cache, size_t seq_stride, const void *d_qabs,
                  void *d_workspace, void *d_o_lat, int32_t batch, int32_t seq, int32_t kernel, void *stream);

/* ---- the decoder stack: generate() / run() (:780-893) ------------------------------------
 * A kx_model owns one HBM arena: seeded random-init weights of cfg->n_layers layers (layer
 * l < first_dense dense, the others MoE), the latent KV cache [layers][max_batch][max_context]
 * and the scratch of one decode step.  Not re-entrant; one private stream; a decode step
 * only enqueues work (expert ids and sampled ids stay on the device).
 * kx_prefill     : run() over the prompt token by token as the reference does (:886), sampling
 *                  on the last prompt token; h_ids u32 [batch][prompt_len]; restarts at position 0.
 * kx_decode_step : one run() at the next position; h_ids u32 [batch], or NULL to feed the ids
 *                  sampled by the previous step (no host round trip).
 * kx_greedy_sample: sample_lm_head (:718-734): lowest-index argmax over the bf16-rounded
 *                  logits of the last step; h_out u32 [batch]; synchronises.
 * kx_generate    : the loops at :885-890; h_out u32 [batch][n_tokens], h_counts i32 [batch] ids
 *                  emitted per sequence (stops before eos_id unless ignore_eos).              */
typedef struct kx_model kx_model;
int kx_model_bytes(const kx_config *cfg, uint64_t *weights, uint64_t *kv_cache, uint64_t *scratch);
int kx_model_create(const kx_config *cfg, kx_model **model);
int kx_model_destroy(kx_model *model);
int kx_prefill(kx_model *model, const uint32_t *h_ids, int32_t batch, int32_t prompt_len);
int kx_decode_step(kx_model *model, const uint32_t *h_ids);
int kx_greedy_sample(kx_model *model, uint32_t *h_out);
int kx_generate(kx_model *model, const uint32_t *h_prompt, int32_t batch, int32_t prompt_len,
                int32_t n_tokens, int ignore_eos, uint32_t *h_out, int32_t *h_counts);
/* ---- checkpoint: runtime-index.blok -> resident weights ----------------------------------------
 * The index is the text file scripts/model_fetch.py materialize() writes (:116-131): a header line
 * `blok-runtime-index-v1`, then one line per checkpoint tensor,
 *   tensor <name> <role> <layer> <expert> <slot> <dtype> <shape> <off> <bytes> <align> <data> <data_bytes> <file>
 * with [off, off+bytes) the 4096-aligned extent of <file> that holds the data range
 * [data, data+data_bytes).  A <file> that is not absolute is taken relative to the index's directory.
 * kx_index_check       : runtime_index() (:559-585) + validate_forward_contract() (:736-778) with the
 *                        shapes of *cfg for layers [0, cfg->n_layers): the tensors the forward pass
 *                        reads and their data bytes.  Needs no GPU.
 * kx_index_infer_config: overwrites the shape fields of *cfg (vocab, hidden, n_layers, first_dense,
 *                        q_rank, kv_rank, heads, dense_inter, experts, shared_inter, moe_inter) with what
 *                        the index's tensor shapes say, and sets yarn_factor to 64, the constant the
 *                        reference computes a checkpoint with (src/kimi_exec.cu:184; kx_config_default's 32
 *                        is for the seeded random-init configurations; set the field afterwards to
 *                        override).  Head dimensions, topk and the other numeric constants are not in a
 *                        checkpoint's shapes and stay as they are.  Needs no GPU.
 * kx_model_load        : a kx_model whose weights are read from the index's files instead of being
 *                        random-init (load_tensor / load_rows, :608-649, which the reference runs per
 *                        tile per token; here once).  kv_b_proj stays whole: its rows h*256+d are
 *                        W_UK[h] for d < 128 and W_UV[h] above (split_kv_k, :364-370).  The router bias
 *                        is widened from bf16 to f32.  KX_LOAD_THREADS (default 8) reader threads;
 *                        KX_LOAD_DIRECT=0 turns O_DIRECT reads off.
 * kx_model_load_info   : data bytes copied by kx_model_load and the seconds it took.               */
int kx_index_check(const kx_config *cfg, const char *index_path, uint64_t *n_tensors, uint64_t *weight_bytes);
int kx_index_infer_config(const char *index_path, kx_config *cfg);
int kx_model_load(const kx_config *cfg, const char *index_path, kx_model **model);
int kx_model_load_info(kx_model *model, uint64_t *bytes, double *seconds);
/* ---- tokenizer.blok: the encoder on the caller's side of the executor (host only, needs no GPU) ----
 * The file is written by scripts/model_fetch.py tokenizer() (:81-97): `blok-tokenizer-v2`, then
 * `tok <id> <hex>` per mergeable byte string and `special <id> <hex>` per special token.
 * kx_tokenizer_open  : tokenizer_encoding() of blok/runtime.py (:121-134); "bad tokenizer" on a malformed file.
 * kx_pretokenize     : the split the pattern KIMI_PATTERN (runtime.py:37-48) makes of UTF-8 `text`:
 *                      h_ends[i] = byte offset where piece i ends.
 * kx_tokenizer_encode: tiktoken's Encoding.encode: with allow_special every special token's text found in
 *                      `text` becomes its id (allowed_special="all", runtime.py:140) and the text between
 *                      is split by the pattern and merged pair by pair, lowest rank first; without it the
 *                      whole text is ordinary.
 * kx_tokenizer_decode: the bytes of the ids, concatenated (Encoding.decode before its UTF-8 step).
 * kx_encode_prompt   : encode_prompt() (runtime.py:137-140): the chat template
 *                      <|im_user|>user<|im_middle|>{prompt}<|im_end|><|im_assistant|>assistant<|im_middle|><think></think>
 * Output buffers: *n (or *len) is always set to the size needed; a buffer that is too small is an error. */
typedef struct kx_tokenizer kx_tokenizer;
int kx_tokenizer_open(const char *path, kx_tokenizer **tok);
int kx_tokenizer_close(kx_tokenizer *tok);
int kx_tokenizer_info(const kx_tokenizer *tok, int32_t *n_tokens, int32_t *n_special, int32_t *max_id);
int kx_pretokenize(const char *text, size_t len, uint32_t *h_ends, size_t cap, size_t *n);
int kx_tokenizer_encode(const kx_tokenizer *tok, const char *text, size_t len, int allow_special, uint32_t *h_ids,
                        size_t cap, size_t *n);
int kx_tokenizer_decode(const kx_tokenizer *tok, const uint32_t *h_ids, size_t n_ids, char *h_bytes, size_t cap, size_t *len);
int kx_encode_prompt(const kx_tokenizer *tok, const char *prompt, size_t len, uint32_t *h_ids, size_t cap, size_t *n);
/* views for parity checks (synchronise): residual stream bf16 [batch][hidden], logits f32
 * [batch][vocab] of the last sampled step, latent cache rows bf16 [n][kv_rank+qk_rope]         */
int kx_model_hidden(kx_model *model, uint16_t *h_out);
int kx_model_logits(kx_model *model, float *h_out);
int kx_model_latent(kx_model *model, int32_t layer, int32_t seq_index, int32_t pos0, int32_t n, uint16_t *h_out);
/* the model's private stream (hipStream_t), for event timing around its entry points          */
int kx_model_stream(kx_model *model, void **stream);
/* ms of GPU time of the last kx_generate: [0] prefill, [1] decode steps                         */
int kx_model_timing(kx_model *model, float *ms2);
/* ids sampled per sequence by the last kx_generate.  With ignore_eos = 0 the loop ends once every sequence has
 * sampled the end-of-sequence id, as the reference's does (src/kimi_exec.cu:887-888); the ids are read back every
 * eighth step for that, so up to seven steps past the last sequence's end are decoded.             */
int kx_model_steps_decoded(kx_model *model, int32_t *steps);
/* Which steps of a decode layer ride inside the launch of the GEMV before them (up to 4 tokens).
 * Results do not depend on the mask (same sums, same rounding points); it exists so that a test
 * can run both forms.  No counterpart in the reference, which launches every step on its own
 * (src/kimi_exec.cu:812-827).  Default KX_FUSE_ALL.                                            */
#define KX_FUSE_ABSORB 1u   /* W_UK absorb, RoPE of q, kv_a norm + cache row: inside the q_b GEMV */
#define KX_FUSE_MOE_TAIL 2u /* one token: shared down GEMV + combine + residual inside the routed down launch */
#define KX_FUSE_FRONT 4u    /* one token, Kimi-K2 shapes, a device with at least 4 * heads CUs: q_a | kv_a, q_b, the absorb, RoPE and
                               the cache row as one resident launch (takes precedence over KX_FUSE_ABSORB) */
#define KX_FUSE_BACK 8u     /* one token, same conditions, up to 32 attention spans: the merge of the attention partials, W_UV and
                               o_proj with the residual add as one resident launch */
#define KX_FUSE_MOE_HEAD 16u /* with KX_FUSE_BACK, in front of a MoE layer (shared_inter = 32 * heads, an even number of at most 510
                               experts): the post-attention norm, the router, the routing and the shared expert's gate/up ride in
                               that launch */
#define KX_FUSE_ROUTED 32u  /* one token, Kimi-K2 shapes, a device with at least 256 CUs, with KX_FUSE_MOE_TAIL: the routed experts' gate/up
                               rides in the launch of their down projection (one resident launch for the routed experts and the tail) */
#define KX_FUSE_ALL 63u
int kx_model_set_fusion(kx_model *model, uint32_t mask);
/* Test hook for the failure path of the resident launches (KX_FUSE_FRONT, _BACK, _MOE_HEAD, _ROUTED): sets the
 * model's device-side flag as a workgroup does that has given a wait for another workgroup's values up.  From then
 * on a workgroup whose first poll does not succeed gives up at once, every launch still ends normally, and the next
 * call that synchronises (kx_greedy_sample, kx_generate) returns KX_ERR_STATE with a message naming
 * kx_model_set_fusion.  The flag stays set: the model is only good for kx_model_destroy afterwards.              */
int kx_model_debug_fail_waits(kx_model *model);
/* The attention kernel this model's steps use: KX_MLA_AUTO (default), KX_MLA_VALU or KX_MLA_MATRIX_CORES, as for
 * kx_mla_decode.  A property of the model: other models of the process keep theirs.                          */
int kx_model_set_attention_kernel(kx_model *model, int32_t kernel);
/* kx_model_set_exact(model, KX_EXACT_ALL): every step takes the kernels of the bit-reproducible path -- the GEMV
 * kernels, the VALU attention kernel, one prompt position per prefill step -- whatever the batch size, instead of
 * moving to the matrix cores from 5 sequences on.  A sequence then comes out to the bit as it does alone (every sum
 * of that path is a fixed tree that does not depend on the batch), at a few times the cost per step for large
 * batches.  The mask selects the parts (so that a deviation can be traced to one of them); 0, the default, none.
 * No counterpart in the reference, whose batch is always 1 (src/kimi_exec.cu:792-799).
 * kx_model_rewind(model, n): the next step runs at a position n lower than it would have: the last n cache rows of
 * every sequence are written again by the steps that follow (rows above the current position are never read).  After
 * a rewind kx_decode_step needs host ids.  What a caller that rejects drafted tokens needs, and what lets a test run
 * the same step twice, once on each path, from the same cache.                                                 */
#define KX_EXACT_PROJECTIONS 1u /* q_a|kv_a, q_b, o_proj, dense MLP, lm_head as GEMVs */
#define KX_EXACT_ATTENTION 2u   /* the VALU attention kernel */
#define KX_EXACT_SHARED 4u      /* the shared expert as GEMVs */
#define KX_EXACT_ROUTED 8u      /* every routed expert through the INT4 GEMV kernels */
#define KX_EXACT_ALL 15u
int kx_model_set_exact(kx_model *model, uint32_t mask);
int kx_model_rewind(kx_model *model, int32_t positions);
/* A record of the routing for tests and measurement.  The reference's host knows the expert ids of every layer
 * (it copies them back, src/kimi_exec.cu:844); here they stay on the device, and this is the way to look at them.
 * kx_model_set_routing_record(model, 1): from now on every step also keeps, per MoE layer, the router logits of its
 * first min(tokens, max_batch) tokens and the number of distinct experts its tokens selected (two small device
 * copies per layer; off by default).
 * kx_model_routing: the record of the last step for `layer`: h_logits f32 [batch][experts] (or NULL), h_distinct
 * i32 [1] (or NULL).  Synchronises.  A dense layer is an error.
 * kx_model_set_routing_record(model, 2) also keeps the router logits of every position of every sequence, whichever
 * step computed them (n_layers x max_context x max_batch x experts floats of device memory), so that a prefill in
 * steps of several positions can be compared with one token by token, position by position.
 * kx_model_routing_history: h_logits f32 [n][max_batch][experts] for positions pos0 .. pos0 + n - 1 of `layer`.   */
int kx_model_set_routing_record(kx_model *model, int on);
int kx_model_routing(kx_model *model, int32_t layer, float *h_logits, int32_t *h_distinct);
int kx_model_routing_history(kx_model *model, int32_t layer, int32_t pos0, int32_t n, float *h_logits);
/* Prompt positions per prefill step.  1 (default) is the reference's prefill, one run() per prompt token (:886),
 * and the bit-reproducible path.  With n > 1, kx_prefill and kx_generate take up to n consecutive positions of
 * every sequence in one step (at most 2048 tokens a step, so min(n, 2048 / batch) positions): the projections, the
 * shared expert and the attention then run on the matrix cores as they do for a batch of that many sequences, and
 * from 33 tokens a step on the routed experts too (the grouped GEMMs of kx_moe_prefill_layer).  Same values, another
 * summation order: logits within the stack-level tolerance of the token-by-token prefill.  Each position attends to
 * the cache rows up to its own, and only the last position is sampled.  1 <= n <= 2048. */
int kx_model_set_prefill_chunk(kx_model *model, int32_t positions);
/* bf(mean + sigma*z) fill used for the norm weights */
int kx_fill_affine_bf16(void *d_out, uint64_t n, uint64_t seed, uint64_t tensor_id, float mean,
                        float sigma, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* KX_H */
