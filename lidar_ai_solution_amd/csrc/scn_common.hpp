// Shared host-side helpers of libscn_hip: logging, error state, HIP call checking, device buffers.
#pragma once

#include <atomic>

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/scn_c_api.h"

namespace scn {

enum LogLevel : int { kVerb = 0, kWarn = 1, kError = 2, kQuiet = 99 };

void log_message(const char* file, int line, int level, const char* fmt, ...) __attribute__((format(printf, 4, 5)));
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

// Debug mode (SCN_DEBUG_SYNC=1 in the environment, or scn_set_debug_sync): every step of a forward and every stage-level
// entry point waits for its kernels and reports an asynchronous failure with the step's name, instead of letting it
// surface at some later call.  Not for captured graphs (it synchronises) and not for timing.
bool debug_sync_enabled();
int debug_sync_check(hipStream_t stream, const char* what);

#define SCN_LOGV(...) ::scn::log_message(__FILE__, __LINE__, ::scn::kVerb, __VA_ARGS__)
#define SCN_LOGW(...) ::scn::log_message(__FILE__, __LINE__, ::scn::kWarn, __VA_ARGS__)
#define SCN_LOGE(...) ::scn::log_message(__FILE__, __LINE__, ::scn::kError, __VA_ARGS__)

// Fails with SCN_ERR_HIP from the enclosing int-returning function when a HIP call fails.
#define SCN_HIP(call)                                                                          \
  do {                                                                                         \
    hipError_t e__ = (call);                                                                   \
    if (e__ != hipSuccess) {                                                                   \
      ::scn::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e__), __FILE__, __LINE__); \
      return SCN_ERR_HIP;                                                                      \
    }                                                                                          \
  } while (0)

#define SCN_REQUIRE(cond, code, ...)  \
  do {                                \
    if (!(cond)) {                    \
      ::scn::set_error(__VA_ARGS__);  \
      return code;                    \
    }                                 \
  } while (0)

// Owning device allocation.  alloc() returns false (and sets the error) on failure.
// Pinned host memory that kernels can write (hipHostMalloc: mapped into the device address space).
struct HostBuf {
  void* p = nullptr;
  HostBuf() = default;
  HostBuf(const HostBuf&) = delete;
  HostBuf& operator=(const HostBuf&) = delete;
  HostBuf(HostBuf&& o) noexcept : p(o.p) { o.p = nullptr; }
  HostBuf& operator=(HostBuf&& o) noexcept {
    if (this != &o) {
      release();
      p = o.p;
      o.p = nullptr;
    }
    return *this;
  }
  ~HostBuf() { release(); }
  bool alloc(size_t n) {
    release();
    if (hipHostMalloc(&p, n ? n : 16, hipHostMallocDefault) != hipSuccess) {
      p = nullptr;
      return false;
    }
    return true;
  }
  void release() {
    if (p) (void)hipHostFree(p);
    p = nullptr;
  }
  template <class T>
  T* as() const {
    return static_cast<T*>(p);
  }
};

// device bytes currently held by DevBuf objects of this process (scn_device_bytes_in_use)
std::atomic<size_t>& device_bytes_counter();

struct DevBuf {
  void* p = nullptr;
  size_t bytes = 0;
  DevBuf() = default;
  DevBuf(const DevBuf&) = delete;
  DevBuf& operator=(const DevBuf&) = delete;
  DevBuf(DevBuf&& o) noexcept : p(o.p), bytes(o.bytes) {
    o.p = nullptr;
    o.bytes = 0;
  }
  DevBuf& operator=(DevBuf&& o) noexcept {
    if (this != &o) {
      release();
      p = o.p;
      bytes = o.bytes;
      o.p = nullptr;
      o.bytes = 0;
    }
    return *this;
  }
  ~DevBuf() { release(); }
  bool alloc(size_t n) {
    release();
    if (n == 0) n = 16;
    hipError_t e = hipMalloc(&p, n);
    if (e != hipSuccess) {
      p = nullptr;
      set_error("hipMalloc(%zu) failed: %s", n, hipGetErrorString(e));
      return false;
    }
    bytes = n;
    device_bytes_counter() += n;
    return true;
  }
  void release() {
    if (p) {
      (void)hipFree(p);
      device_bytes_counter() -= bytes;
    }
    p = nullptr;
    bytes = 0;
  }
  template <typename T>
  T* as() const {
    return reinterpret_cast<T*>(p);
  }
};

inline uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

// fp16 bits <-> float on the host (round to nearest even), used when packing weights.
float half_bits_to_float(uint16_t h);
uint16_t float_to_half_bits(float f);

}  // namespace scn
