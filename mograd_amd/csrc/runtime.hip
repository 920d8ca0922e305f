// Library plumbing: error state, device properties, streams and the caching pool.
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "mg_device.h"
#include "mg_internal.h"

namespace mg {

template <typename T>
__global__ void fill_kernel(T* dst, T value, int64_t n) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    dst[i] = value;
}

template <typename T>
static int launch_fill(void* dst, T value, int64_t n, hipStream_t stream) {
  int64_t blocks = ceil_div(n, 256);
  const int64_t cap = static_cast<int64_t>(device_info().cu_count) * 16;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL((fill_kernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, static_cast<T*>(dst),
                     value, n);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

// ------------------------------------------------------------------------------------
// Errors
// ------------------------------------------------------------------------------------

static thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

void clear_error() { g_last_error.clear(); }

// ------------------------------------------------------------------------------------
// Device properties
// ------------------------------------------------------------------------------------

static std::mutex g_info_mu;
static std::unordered_map<int, DeviceInfo> g_info;

const DeviceInfo& device_info() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  std::lock_guard<std::mutex> lock(g_info_mu);
  auto it = g_info.find(dev);
  if (it != g_info.end()) return it->second;
  DeviceInfo info;
  info.device = dev;
  int v = 0;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess) info.cu_count = v;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxThreadsPerBlock, dev) == hipSuccess) info.max_threads = v;
  if (info.cu_count <= 0) info.cu_count = 256;
  if (info.max_threads <= 0) info.max_threads = 1024;
  return g_info.emplace(dev, info).first->second;
}

// ------------------------------------------------------------------------------------
// Pool.  Size classes and counters follow mograd/memory.mojo:59-105,242-311,353-362.
// One pool per device; a block remembers its class so release needs only the pointer.
// ------------------------------------------------------------------------------------

static int64_t round_class(int64_t nbytes) {
  constexpr int64_t kMinClass = 512;
  constexpr int64_t kDivisions = 8;
  if (nbytes <= kMinClass) return kMinClass;
  int64_t p = 1;
  while ((p << 1) <= nbytes) p <<= 1;
  if (p == nbytes) return nbytes;
  int64_t step = p / kDivisions;
  return ((nbytes + step - 1) / step) * step;
}

struct Pool {
  std::unordered_map<int64_t, std::vector<void*>> free_lists;
  std::unordered_map<void*, int64_t> live;  // ptr -> class bytes (pooled) or -nbytes (unpooled)
  mg_pool_stats stats{};
};

static std::mutex g_pool_mu;
static std::unordered_map<int, Pool> g_pools;

static bool pool_enabled_env() {
  static const bool enabled = [] {
    const char* v = std::getenv("MOGRAD_POOL");
    return !(v && std::strcmp(v, "0") == 0);
  }();
  return enabled;
}

static Pool& current_pool() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  return g_pools[dev];
}

static void empty_cache_locked(Pool& pool) {
  for (auto& kv : pool.free_lists)
    for (void* p : kv.second) (void)hipFree(p);
  pool.free_lists.clear();
  pool.stats.reserved_bytes = pool.stats.allocated_bytes;
}

static std::string fmt_bytes(int64_t n) {
  char buf[64];
  if (n < 1024) {
    snprintf(buf, sizeof(buf), "%lld B", static_cast<long long>(n));
    return buf;
  }
  const char* unit = "KiB";
  int64_t div = int64_t(1) << 10;
  if (n >= (int64_t(1) << 30)) {
    unit = "GiB";
    div = int64_t(1) << 30;
  } else if (n >= (int64_t(1) << 20)) {
    unit = "MiB";
    div = int64_t(1) << 20;
  }
  int64_t tenths = (n * 10) / div;
  snprintf(buf, sizeof(buf), "%lld.%lld %s", static_cast<long long>(tenths / 10),
           static_cast<long long>(tenths % 10), unit);
  return buf;
}

static std::string summary_locked(Pool& pool) {
  const mg_pool_stats& s = pool.stats;
  std::string out = "mograd memory pool:\n";
  out += "  allocated: " + fmt_bytes(s.allocated_bytes) + "  (peak " + fmt_bytes(s.peak_allocated) + ")\n";
  out += "  reserved:  " + fmt_bytes(s.reserved_bytes) + "  (peak " + fmt_bytes(s.peak_reserved) + ")\n";
  out += "  counters:  " + std::to_string(s.alloc_count) + " driver allocs | " + std::to_string(s.hit_count) +
         " hits | " + std::to_string(s.miss_count) + " misses | " + std::to_string(s.free_count) + " frees\n";
  int classes = 0;
  int64_t blocks = 0;
  std::string census;
  for (auto& kv : pool.free_lists) {
    if (kv.second.empty()) continue;
    ++classes;
    blocks += static_cast<int64_t>(kv.second.size());
    census += "    " + fmt_bytes(kv.first) + " x " + std::to_string(kv.second.size()) + "\n";
  }
  out += "  free lists (" + std::to_string(classes) + " classes, " + std::to_string(blocks) + " blocks):\n";
  out += census;
  return out;
}

int pool_take(void** out, int64_t nbytes) {
  if (!out) return fail(MG_ERR_INVALID, "pool_alloc: null output pointer");
  if (nbytes < 0) return fail(MG_ERR_INVALID, "pool_alloc: negative size %lld", static_cast<long long>(nbytes));
  *out = nullptr;
  std::lock_guard<std::mutex> lock(g_pool_mu);
  Pool& pool = current_pool();
  if (!pool_enabled_env()) {
    void* p = nullptr;
    int64_t n = nbytes > 0 ? nbytes : 1;
    hipError_t e = hipMalloc(&p, static_cast<size_t>(n));
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return fail(MG_ERR_OOM, "mograd: out of device memory allocating %s", fmt_bytes(n).c_str());
    }
    pool.live[p] = -n;
    *out = p;
    return MG_OK;
  }
  const int64_t cls = round_class(nbytes);
  void* p = nullptr;
  auto it = pool.free_lists.find(cls);
  if (it != pool.free_lists.end() && !it->second.empty()) {
    p = it->second.back();
    it->second.pop_back();
    pool.stats.hit_count += 1;
  } else {
    hipError_t e = hipMalloc(&p, static_cast<size_t>(cls));
    if (e != hipSuccess) {
      // Out of memory: release every cached block, wait for the device, retry once.
      (void)hipGetLastError();
      empty_cache_locked(pool);
      (void)hipDeviceSynchronize();
      e = hipMalloc(&p, static_cast<size_t>(cls));
      if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(MG_ERR_OOM, "mograd: out of device memory allocating %s\n%s", fmt_bytes(cls).c_str(),
                    summary_locked(pool).c_str());
      }
    }
    pool.stats.miss_count += 1;
    pool.stats.alloc_count += 1;
    pool.stats.reserved_bytes += cls;
  }
  pool.live[p] = cls;
  mg_pool_stats& s = pool.stats;
  s.allocated_bytes += cls;
  if (s.allocated_bytes > s.peak_allocated) s.peak_allocated = s.allocated_bytes;
  if (s.reserved_bytes > s.peak_reserved) s.peak_reserved = s.reserved_bytes;
  *out = p;
  return MG_OK;
}

int pool_release(void* ptr) {
  if (!ptr) return MG_OK;
  std::lock_guard<std::mutex> lock(g_pool_mu);
  Pool& pool = current_pool();
  auto it = pool.live.find(ptr);
  if (it == pool.live.end()) return fail(MG_ERR_INVALID, "pool_free: pointer %p was not allocated by this pool", ptr);
  const int64_t cls = it->second;
  pool.live.erase(it);
  if (cls < 0) {  // unpooled: plain release (hipFree waits for the device)
    (void)hipFree(ptr);
    return MG_OK;
  }
  pool.free_lists[cls].push_back(ptr);
  pool.stats.allocated_bytes -= cls;
  pool.stats.free_count += 1;
  return MG_OK;
}

}  // namespace mg

// ------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------

extern "C" {

const char* mg_version(void) { return "mograd_hip 0.1 (gfx950)"; }

const char* mg_last_error(void) { return mg::g_last_error.c_str(); }

int mg_init(int device) {
  MG_HIP(hipSetDevice(device));
  (void)mg::device_info();
  // The static scratch of the non-allocating entry point: resolve this device's copy now, so
  // that its first call does no set-up work.  A failure here (a device ordinal beyond its
  // table, say) concerns that one optional entry point, which reports it when called: the rest
  // of the library stays usable.
  if (mg::ce_noalloc_setup(nullptr) != MG_OK) mg::clear_error();
  return MG_OK;
}

int mg_device_cu_count(void) { return mg::device_info().cu_count; }

int mg_stream_create(mg_stream* out) {
  if (!out) return mg::fail(MG_ERR_INVALID, "stream_create: null output pointer");
  hipStream_t s = nullptr;
  MG_HIP(hipStreamCreate(&s));
  *out = s;
  return MG_OK;
}

int mg_stream_destroy(mg_stream stream) {
  if (!stream) return MG_OK;
  MG_HIP(hipStreamDestroy(mg::to_stream(stream)));
  return MG_OK;
}

int mg_stream_sync(mg_stream stream) {
  MG_HIP(hipStreamSynchronize(mg::to_stream(stream)));
  return MG_OK;
}

int mg_event_create(mg_event* out) {
  if (!out) return mg::fail(MG_ERR_INVALID, "event_create: null output pointer");
  hipEvent_t e = nullptr;
  MG_HIP(hipEventCreate(&e));
  *out = e;
  return MG_OK;
}

int mg_event_destroy(mg_event event) {
  if (!event) return MG_OK;
  MG_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return MG_OK;
}

int mg_event_record(mg_event event, mg_stream stream) {
  if (!event) return mg::fail(MG_ERR_INVALID, "event_record: null event");
  MG_HIP(hipEventRecord(static_cast<hipEvent_t>(event), mg::to_stream(stream)));
  return MG_OK;
}

int mg_event_elapsed_ms(mg_event start, mg_event stop, float* ms) {
  if (!start || !stop || !ms) return mg::fail(MG_ERR_INVALID, "event_elapsed_ms: null argument");
  MG_HIP(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
  MG_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return MG_OK;
}

int mg_copy_to_device(void* dst, const void* host_src, int64_t nbytes, mg_stream stream) {
  if (nbytes < 0 || (nbytes > 0 && (!dst || !host_src))) return mg::fail(MG_ERR_INVALID, "copy_to_device: bad argument");
  if (nbytes == 0) return MG_OK;
  MG_HIP(hipMemcpyAsync(dst, host_src, static_cast<size_t>(nbytes), hipMemcpyHostToDevice, mg::to_stream(stream)));
  MG_HIP(hipStreamSynchronize(mg::to_stream(stream)));
  return MG_OK;
}

int mg_copy_to_host(void* host_dst, const void* src, int64_t nbytes, mg_stream stream) {
  if (nbytes < 0 || (nbytes > 0 && (!host_dst || !src))) return mg::fail(MG_ERR_INVALID, "copy_to_host: bad argument");
  if (nbytes == 0) return MG_OK;
  MG_HIP(hipMemcpyAsync(host_dst, src, static_cast<size_t>(nbytes), hipMemcpyDeviceToHost, mg::to_stream(stream)));
  MG_HIP(hipStreamSynchronize(mg::to_stream(stream)));
  return MG_OK;
}

int mg_copy_device(void* dst, const void* src, int64_t nbytes, mg_stream stream) {
  if (nbytes < 0 || (nbytes > 0 && (!dst || !src))) return mg::fail(MG_ERR_INVALID, "copy_device: bad argument");
  if (nbytes == 0) return MG_OK;
  MG_HIP(hipMemcpyAsync(dst, src, static_cast<size_t>(nbytes), hipMemcpyDeviceToDevice, mg::to_stream(stream)));
  return MG_OK;
}

int mg_fill(void* dst, double value, int64_t numel, int dtype, mg_stream stream) {
  if (numel < 0 || (numel > 0 && !dst)) return mg::fail(MG_ERR_INVALID, "fill: bad argument");
  if (numel == 0) return MG_OK;
  hipStream_t s = mg::to_stream(stream);
  switch (dtype) {
    case MG_F32: return mg::launch_fill<float>(dst, static_cast<float>(value), numel, s);
    case MG_F16: return mg::launch_fill<_Float16>(dst, static_cast<_Float16>(value), numel, s);
    case MG_BF16: {
      // Round to nearest even on the host.
      float f = static_cast<float>(value);
      uint32_t u;
      std::memcpy(&u, &f, sizeof(u));
      if ((u & 0x7fffffffu) > 0x7f800000u) u = (u >> 16) | 0x40u;
      else u = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
      return mg::launch_fill<uint16_t>(dst, static_cast<uint16_t>(u), numel, s);
    }
    case MG_I32: return mg::launch_fill<int32_t>(dst, static_cast<int32_t>(value), numel, s);
    case MG_I64: return mg::launch_fill<int64_t>(dst, static_cast<int64_t>(value), numel, s);
    default: return mg::fail(MG_ERR_INVALID, "fill: unsupported dtype %d", dtype);
  }
}

int64_t mg_round_class(int64_t nbytes) { return mg::round_class(nbytes); }

int mg_pool_enabled(void) { return mg::pool_enabled_env() ? 1 : 0; }

int mg_pool_alloc(void** out, int64_t nbytes) { return mg::pool_take(out, nbytes); }

int mg_pool_free(void* ptr) { return mg::pool_release(ptr); }

int mg_pool_empty_cache(void) {
  std::lock_guard<std::mutex> lock(mg::g_pool_mu);
  mg::empty_cache_locked(mg::current_pool());
  return MG_OK;
}

int mg_pool_get_stats(mg_pool_stats* out) {
  if (!out) return mg::fail(MG_ERR_INVALID, "pool_get_stats: null output pointer");
  std::lock_guard<std::mutex> lock(mg::g_pool_mu);
  *out = mg::current_pool().stats;
  return MG_OK;
}

int64_t mg_pool_summary(char* buf, int64_t cap) {
  std::lock_guard<std::mutex> lock(mg::g_pool_mu);
  std::string s = mg::summary_locked(mg::current_pool());
  if (buf && cap > 0) {
    int64_t n = static_cast<int64_t>(s.size()) < cap - 1 ? static_cast<int64_t>(s.size()) : cap - 1;
    std::memcpy(buf, s.data(), static_cast<size_t>(n));
    buf[n] = '\0';
  }
  return static_cast<int64_t>(s.size());
}

}  // extern "C"
