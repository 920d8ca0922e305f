// Host-side internals shared by every translation unit of libmograd_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>

#include "mograd_hip.h"

namespace mg {

// Records `msg` as this thread's last error and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

struct DeviceInfo {
  int device = -1;
  int cu_count = 0;
  int max_threads = 0;
};
// Properties of the current device, read once per device.
const DeviceInfo& device_info();

// cross_entropy.hip: address of the current device's static per-row loss scratch (resolved
// on the first call per device); `out` may be null.
int ce_noalloc_setup(float** out);

// Pool (runtime.hip).  Thread-safe; see mg_pool_alloc / mg_pool_free.
int pool_take(void** out, int64_t nbytes);
int pool_release(void* ptr);

// A scratch buffer from the pool, returned when the object dies.  Work that uses it has
// already been enqueued on the caller's stream by then; the block is only handed out to
// later calls, which enqueue behind that work on the same stream.
class Scratch {
 public:
  Scratch() = default;
  ~Scratch() {
    if (ptr_) pool_release(ptr_);
  }
  Scratch(const Scratch&) = delete;
  Scratch& operator=(const Scratch&) = delete;
  int take(int64_t nbytes) { return pool_take(&ptr_, nbytes); }
  // Gives the block up without returning it to the pool: the caller now owns it.
  void* detach() {
    void* p = ptr_;
    ptr_ = nullptr;
    return p;
  }
  template <typename T>
  T* as() const {
    return static_cast<T*>(ptr_);
  }

 private:
  void* ptr_ = nullptr;
};

// A view of up to kMaxRank dimensions: extents and element strides, passed to kernels by
// value.
constexpr int kMaxRank = 8;
struct StridedView {
  int rank;
  int64_t shape[kMaxRank];
  int64_t stride[kMaxRank];
};

inline hipStream_t to_stream(mg_stream s) { return static_cast<hipStream_t>(s); }

inline bool is_float_dtype(int dtype) { return dtype == MG_F32 || dtype == MG_F16 || dtype == MG_BF16; }
inline int dtype_size(int dtype) {
  switch (dtype) {
    case MG_F32: return 4;
    case MG_F16: return 2;
    case MG_BF16: return 2;
    case MG_I32: return 4;
    case MG_I64: return 8;
    default: return 0;
  }
}
inline const char* dtype_name(int dtype) {
  switch (dtype) {
    case MG_F32: return "float32";
    case MG_F16: return "float16";
    case MG_BF16: return "bfloat16";
    case MG_I32: return "int32";
    case MG_I64: return "int64";
    default: return "?";
  }
}

// The MOGRAD_HIP_* tuning knobs (kernel layout choices that benchmarks and equivalence tests
// flip without rebuilding) are honoured only in a process that sets MOGRAD_HIP_TUNING=1, so
// that the library's behaviour in a host application does not depend on stray variables of
// its environment.  Read once.
inline bool tuning_enabled() {
  static const bool on = [] {
    const char* v = std::getenv("MOGRAD_HIP_TUNING");
    return v && v[0] == '1';
  }();
  return on;
}
// A tuning knob's raw value, or null when unset or when tuning is off.
inline const char* env_str(const char* name) {
  if (!tuning_enabled()) return nullptr;
  const char* v = std::getenv(name);
  return (v && *v) ? v : nullptr;
}
// Integer tuning knob (looked up on every call).
inline int env_int(const char* name, int fallback) {
  const char* v = env_str(name);
  return v ? std::atoi(v) : fallback;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace mg

#define MG_HIP(expr)                                                                        \
  do {                                                                                      \
    hipError_t mg_e_ = (expr);                                                              \
    if (mg_e_ != hipSuccess)                                                                \
      return ::mg::fail(MG_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(mg_e_), \
                        __FILE__, __LINE__);                                                \
  } while (0)

#define MG_TRY(expr)            \
  do {                          \
    int mg_rc_ = (expr);        \
    if (mg_rc_ != 0) return mg_rc_; \
  } while (0)

// After a kernel launch: surfaces launch-configuration errors without synchronising.
#define MG_LAUNCH_CHECK() MG_HIP(hipGetLastError())
