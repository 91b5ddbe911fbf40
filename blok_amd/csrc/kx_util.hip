// kx_util.hip -- error state, device plumbing and the synthetic-tensor fill kernels.
// Replaces the reference's Buf/DeviceTensor RAII wrappers (src/kimi_exec.cu:137-174)
// and its uGDS tile loaders (:608-649): weights are generated in place in HBM.
#include <stdarg.h>
#include <string.h>
#include "kx_common.h"
#include "kx_rng.h"

static thread_local char g_err[512] = "";

void kx_set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
}

extern "C" const char *kx_last_error(void) { return g_err; }

extern "C" int kx_config_default(kx_config *c) {
  KX_REQUIRE(c, "kx_config_default: null config");
  memset(c, 0, sizeof *c);
  c->n_layers = 24; c->first_dense = 1;
  c->hidden = 7168; c->heads = 64; c->qk_nope = 128; c->qk_rope = 64; c->v_head = 128;
  c->q_rank = 1536; c->kv_rank = 512; c->experts = 384; c->topk = 8;
  c->moe_inter = 2048; c->shared_inter = 2048; c->dense_inter = 18432; c->vocab = 163840;
  c->max_batch = 1; c->max_context = 4096; c->eos_id = 163586u;
  c->rms_eps = 1.0e-5f; c->rope_theta = 50000.0f; c->routed_scale = 2.827f;
  c->yarn_factor = 32.0f; c->yarn_beta_fast = 32.0f; c->yarn_beta_slow = 1.0f;
  c->yarn_orig_ctx = 4096.0f; c->yarn_mscale_all_dim = 1.0f; c->init_sigma = 0.02f; c->expert_scale_sigma = 0.02f;
  c->seed = 0;
  return KX_OK;
}

extern "C" int kx_device_info(char *name, size_t name_len, int32_t *cus, uint64_t *hbm) {
  hipDeviceProp_t p;
  int dev = 0;
  KX_HIP(hipGetDevice(&dev));
  KX_HIP(hipGetDeviceProperties(&p, dev));
  if (name && name_len) {
    snprintf(name, name_len, "%s (%s)", p.name, p.gcnArchName);
  }
  if (cus) *cus = p.multiProcessorCount;
  if (hbm) *hbm = p.totalGlobalMem;
  return KX_OK;
}

extern "C" int kx_dev_malloc(void **d_ptr, size_t bytes) {
  KX_REQUIRE(d_ptr, "kx_dev_malloc: null out pointer");
  *d_ptr = nullptr;
  KX_HIP(hipMalloc(d_ptr, bytes ? bytes : 1));
  return KX_OK;
}
extern "C" int kx_dev_free(void *d_ptr) {
  if (d_ptr) KX_HIP(hipFree(d_ptr));
  return KX_OK;
}
extern "C" int kx_dev_memset(void *d_ptr, int value, size_t bytes, void *stream) {
  KX_REQUIRE(d_ptr || !bytes, "kx_dev_memset: null pointer");
  KX_HIP(hipMemsetAsync(d_ptr, value, bytes, kx_stream(stream)));
  return KX_OK;
}
extern "C" int kx_dev_mem_info(size_t *free_bytes, size_t *total_bytes) {
  KX_REQUIRE(free_bytes && total_bytes, "kx_dev_mem_info: null pointer");
  KX_HIP(hipMemGetInfo(free_bytes, total_bytes));
  return KX_OK;
}
extern "C" int kx_h2d(void *d_dst, const void *h_src, size_t bytes) {
  KX_REQUIRE((d_dst && h_src) || !bytes, "kx_h2d: null pointer");
  KX_HIP(hipMemcpy(d_dst, h_src, bytes, hipMemcpyHostToDevice));
  return KX_OK;
}
extern "C" int kx_d2h(void *h_dst, const void *d_src, size_t bytes) {
  KX_REQUIRE((h_dst && d_src) || !bytes, "kx_d2h: null pointer");
  KX_HIP(hipMemcpy(h_dst, d_src, bytes, hipMemcpyDeviceToHost));
  return KX_OK;
}
extern "C" int kx_sync(void *stream) {
  if (stream) KX_HIP(hipStreamSynchronize(kx_stream(stream)));
  else KX_HIP(hipDeviceSynchronize());
  return KX_OK;
}
extern "C" int kx_event_create(void **event) {
  KX_REQUIRE(event, "kx_event_create: null out pointer");
  hipEvent_t e;
  KX_HIP(hipEventCreate(&e));
  *event = (void *)e;
  return KX_OK;
}
extern "C" int kx_event_destroy(void *event) {
  if (event) KX_HIP(hipEventDestroy((hipEvent_t)event));
  return KX_OK;
}
extern "C" int kx_event_record(void *event, void *stream) {
  KX_REQUIRE(event, "kx_event_record: null event");
  KX_HIP(hipEventRecord((hipEvent_t)event, kx_stream(stream)));
  return KX_OK;
}
extern "C" int kx_event_elapsed_ms(void *start, void *stop, float *ms) {
  KX_REQUIRE(start && stop && ms, "kx_event_elapsed_ms: null argument");
  KX_HIP(hipEventSynchronize((hipEvent_t)stop));
  KX_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return KX_OK;
}

// ---- fill kernels ---------------------------------------------------------------
namespace {
__global__ void fill_normal_bf16_k(uint16_t *out, uint64_t n, uint64_t key, float sigma, int absval) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = kx_rng_normal_bf16(key, i, sigma, absval);
}
__global__ void fill_affine_bf16_k(uint16_t *out, uint64_t n, uint64_t key, float mean, float sigma) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = kx_bf16_rne(mean + kx_rng_normal_f32(key, i, sigma));
}
__global__ void fill_normal_f32_k(float *out, uint64_t n, uint64_t key, float sigma) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = kx_rng_normal_f32(key, i, sigma);
}
__global__ void fill_words_k(uint32_t *out, uint64_t n, uint64_t key) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = kx_rng_u32(key, i);
}
__global__ void fill_tokens_k(uint32_t *out, uint64_t n, uint64_t key, uint32_t vocab) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = (uint32_t)(kx_rng_u64(key, i) % vocab);
}
unsigned fill_grid(uint64_t n) {
  uint64_t b = (n + 255) / 256;
  return (unsigned)(b < 1 ? 1 : (b > 65536 ? 65536 : b));
}
}  // namespace

extern "C" int kx_fill_normal_bf16(void *d_out, uint64_t n, uint64_t seed, uint64_t tensor_id, float sigma,
                                   int absval, void *stream) {
  KX_REQUIRE(d_out || !n, "kx_fill_normal_bf16: null pointer");
  if (!n) return KX_OK;
  hipLaunchKernelGGL(fill_normal_bf16_k, dim3(fill_grid(n)), dim3(256), 0, kx_stream(stream), (uint16_t *)d_out, n,
                     kx_rng_key(seed, tensor_id), sigma, absval);
  KX_LAUNCH_CHECK();
  return KX_OK;
}
extern "C" int kx_fill_normal_f32(void *d_out, uint64_t n, uint64_t seed, uint64_t tensor_id, float sigma,
                                  void *stream) {
  KX_REQUIRE(d_out || !n, "kx_fill_normal_f32: null pointer");
  if (!n) return KX_OK;
  hipLaunchKernelGGL(fill_normal_f32_k, dim3(fill_grid(n)), dim3(256), 0, kx_stream(stream), (float *)d_out, n,
                     kx_rng_key(seed, tensor_id), sigma);
  KX_LAUNCH_CHECK();
  return KX_OK;
}
// plain 16-byte-per-lane copy: the known-traffic kernel that HBM counters are calibrated against
__global__ void __launch_bounds__(256) copy16_k(uint4 *__restrict__ dst, const uint4 *__restrict__ src, uint64_t n16) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * 256) dst[i] = src[i];
}
extern "C" int kx_dev_copy(void *d_dst, const void *d_src, uint64_t bytes, void *stream) {
  KX_REQUIRE((d_dst && d_src) || !bytes, "kx_dev_copy: null pointer");
  KX_REQUIRE(bytes % 16 == 0 && ((uintptr_t)d_dst | (uintptr_t)d_src) % 16 == 0, "kx_dev_copy: 16-byte granularity");
  if (!bytes) return KX_OK;
  hipLaunchKernelGGL(copy16_k, dim3(fill_grid(bytes / 16)), dim3(256), 0, kx_stream(stream), (uint4 *)d_dst,
                     (const uint4 *)d_src, bytes / 16);
  KX_LAUNCH_CHECK();
  return KX_OK;
}
extern "C" int kx_fill_words_u32(void *d_out, uint64_t n, uint64_t seed, uint64_t tensor_id, void *stream) {
  KX_REQUIRE(d_out || !n, "kx_fill_words_u32: null pointer");
  if (!n) return KX_OK;
  hipLaunchKernelGGL(fill_words_k, dim3(fill_grid(n)), dim3(256), 0, kx_stream(stream), (uint32_t *)d_out, n,
                     kx_rng_key(seed, tensor_id));
  KX_LAUNCH_CHECK();
  return KX_OK;
}
extern "C" int kx_fill_tokens_u32(void *d_out, uint64_t n, uint64_t seed, uint64_t tensor_id, uint32_t vocab, void *stream) {
  KX_REQUIRE(d_out || !n, "kx_fill_tokens_u32: null pointer");
  KX_REQUIRE(vocab > 0, "kx_fill_tokens_u32: vocab must be positive");
  if (!n) return KX_OK;
  hipLaunchKernelGGL(fill_tokens_k, dim3(fill_grid(n)), dim3(256), 0, kx_stream(stream), (uint32_t *)d_out, n,
                     kx_rng_key(seed, tensor_id), vocab);
  KX_LAUNCH_CHECK();
  return KX_OK;
}
extern "C" int kx_fill_affine_bf16(void *d_out, uint64_t n, uint64_t seed, uint64_t tensor_id, float mean, float sigma,
                                   void *stream) {
  KX_REQUIRE(d_out || !n, "kx_fill_affine_bf16: null pointer");
  if (!n) return KX_OK;
  hipLaunchKernelGGL(fill_affine_bf16_k, dim3(fill_grid(n)), dim3(256), 0, kx_stream(stream), (uint16_t *)d_out, n,
                     kx_rng_key(seed, tensor_id), mean, sigma);
  KX_LAUNCH_CHECK();
  return KX_OK;
}
