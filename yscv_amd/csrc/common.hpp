// Shared host-side plumbing for the yscv_hip library: status codes, thread-local
// error text, HIP call checking, the device context.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>

#include "../../include/yscv_hip.h"

namespace yscv {

// ---- errors ------------------------------------------------------------------
std::string &last_error_slot();
int32_t set_error(int32_t code, const char *fmt, ...);

#define YSCV_REQUIRE(cond, ...)                                             \
  do {                                                                      \
    if (!(cond)) return ::yscv::set_error(YSCV_HIP_ERR_INVALID_ARG, __VA_ARGS__); \
  } while (0)

#define YSCV_HIP_TRY(expr)                                                            \
  do {                                                                                \
    hipError_t _e = (expr);                                                           \
    if (_e != hipSuccess) {                                                           \
      int32_t _c = (_e == hipErrorOutOfMemory) ? YSCV_HIP_ERR_OOM : YSCV_HIP_ERR_DEVICE; \
      return ::yscv::set_error(_c, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), \
                               __FILE__, __LINE__);                                   \
    }                                                                                 \
  } while (0)

#define YSCV_TRY(expr)          \
  do {                          \
    int32_t _s = (expr);        \
    if (_s != YSCV_HIP_OK) return _s; \
  } while (0)

// ---- context -------------------------------------------------------------------
struct Context {
  int device = -1;
  int num_cus = 0;
  int lds_bytes = 0;
  char arch[64] = {0};
  char name[128] = {0};
  size_t total_mem = 0;
};

// Lazily initialises the context on device 0 (or returns the existing one).
int32_t ensure_context(const Context **out);
int32_t init_context(int device);
void drop_context();

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// RAII device buffer for the host-pointer entry points.
struct DevBuf {
  void *p = nullptr;
  ~DevBuf() {
    if (p) (void)hipFree(p);
  }
  int32_t alloc(size_t bytes) {
    if (bytes == 0) bytes = 4;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess)
      return set_error(e == hipErrorOutOfMemory ? YSCV_HIP_ERR_OOM : YSCV_HIP_ERR_DEVICE,
                       "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    return YSCV_HIP_OK;
  }
  template <typename T>
  T *as() const {
    return static_cast<T *>(p);
  }
};

// Scratch from the stream-ordered allocator: allocation and release are queued on the stream like the kernels that
// use the memory, so the call that owns the buffer can return without waiting for the device.
struct StreamBuf {
  void *p = nullptr;
  hipStream_t s = nullptr;
  ~StreamBuf() {
    if (p) (void)hipFreeAsync(p, s);
  }
  int32_t alloc(size_t bytes, hipStream_t stream) {
    if (bytes == 0) bytes = 4;
    s = stream;
    hipError_t e = hipMallocAsync(&p, bytes, s);
    if (e != hipSuccess) {
      p = nullptr;
      return set_error(e == hipErrorOutOfMemory ? YSCV_HIP_ERR_OOM : YSCV_HIP_ERR_DEVICE,
                       "hipMallocAsync(%zu) failed: %s", bytes, hipGetErrorString(e));
    }
    return YSCV_HIP_OK;
  }
  template <typename T>
  T *as() const {
    return static_cast<T *>(p);
  }
};

inline size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }
inline size_t round_up(size_t a, size_t b) { return ceil_div(a, b) * b; }

}  // namespace yscv
