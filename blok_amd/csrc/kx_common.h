// kx_common.h -- error plumbing shared by the translation units of libkx.
// The reference wraps every CUDA call in ck() and exits (src/kimi_exec.cu:500-502);
// here the same checks set a thread-local message and return a code.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/kx.h"

#define KX_OK 0
#define KX_ERR_ARG 1
#define KX_ERR_HIP 2
#define KX_ERR_STATE 3

void kx_set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define KX_HIP(call)                                                                      \
  do {                                                                                    \
    hipError_t kx_e_ = (call);                                                            \
    if (kx_e_ != hipSuccess) {                                                            \
      kx_set_error("%s: %s (%s:%d)", #call, hipGetErrorString(kx_e_), __FILE__, __LINE__); \
      return KX_ERR_HIP;                                                                  \
    }                                                                                     \
  } while (0)

#define KX_REQUIRE(cond, ...)    \
  do {                           \
    if (!(cond)) {               \
      kx_set_error(__VA_ARGS__); \
      return KX_ERR_ARG;         \
    }                            \
  } while (0)

#define KX_LAUNCH_CHECK() KX_HIP(hipGetLastError())

// No exception may cross the C ABI: the host-side entry points that parse files or grow containers run their
// bodies under this guard (std::bad_alloc from a hostile size, std::out_of_range from a lookup).
#ifdef __cplusplus
#include <exception>
#include <new>
template <class F>
static inline int kx_guard(const char *who, F &&body) {
  try {
    return body();
  } catch (const std::bad_alloc &) {
    kx_set_error("%s: out of memory", who);
  } catch (const std::exception &e) {
    kx_set_error("%s: %s", who, e.what());
  } catch (...) {
    kx_set_error("%s: unknown exception", who);
  }
  return KX_ERR_STATE;
}
#endif

static inline hipStream_t kx_stream(void *s) { return (hipStream_t)s; }
static inline int kx_cdiv(int a, int b) { return (a + b - 1) / b; }

// CUs of the current device (0 when the query fails), remembered per device: the launchers of the resident kernels
// ask before every launch whether all their workgroups fit on the device at once.
static inline int kx_device_cus() {
  static int cus[16];
  int dev = 0, v = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 16 && cus[dev]) return cus[dev];
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) return 0;
  if (dev >= 0 && dev < 16) cus[dev] = v;
  return v;
}
