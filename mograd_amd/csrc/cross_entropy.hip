// C ABI for softmax cross-entropy: argument checks and dtype dispatch.
#include <mutex>

#include "mg_internal.h"

namespace mg {

#define MG_DECLARE_CROSS_ENTROPY(SUFFIX)                                                                         \
  int ce_run_##SUFFIX(bool, const void*, const void*, const void*, void*, void*, int64_t, int64_t, int,          \
                      hipStream_t, float*);                                                                            \
  int ce_run_strided_##SUFFIX(const void*, const void*, const void*, void*, void*, int64_t, int64_t,             \
                              const StridedView&, const StridedView&, hipStream_t);
MG_DECLARE_CROSS_ENTROPY(f32)
MG_DECLARE_CROSS_ENTROPY(f16)
MG_DECLARE_CROSS_ENTROPY(bf16)
#undef MG_DECLARE_CROSS_ENTROPY

static int check_ce(const char* who, int64_t N, int64_t C, int dtype) {
  if (!is_float_dtype(dtype)) return fail(MG_ERR_INVALID, "%s: unsupported dtype %s", who, dtype_name(dtype));
  if (N <= 0 || C <= 0)
    return fail(MG_ERR_INVALID, "%s: bad shape N=%lld C=%lld", who, static_cast<long long>(N), static_cast<long long>(C));
  if (N > 0x7fffffffLL || C > 0x3fffffffLL)
    return fail(MG_ERR_INVALID, "%s: N=%lld or C=%lld exceeds the supported extent", who, static_cast<long long>(N),
                static_cast<long long>(C));
  return MG_OK;
}

static int ce_run(const char* who, bool dense, const void* logits, const void* labels, const void* upstream, void* loss,
                  void* dlogits, int64_t N, int64_t C, int dtype, int id_dtype, mg_stream stream,
                  float* rowloss_ext = nullptr) {
  MG_TRY(check_ce(who, N, C, dtype));
  if (!logits || !labels || (!loss && !dlogits)) return fail(MG_ERR_INVALID, "%s: null pointer argument", who);
  int id64 = 0;
  if (!dense) {
    if (id_dtype != MG_I32 && id_dtype != MG_I64)
      return fail(MG_ERR_INVALID, "%s: ids must be int32 or int64, got %s", who, dtype_name(id_dtype));
    id64 = id_dtype == MG_I64;
  }
  hipStream_t s = to_stream(stream);
  switch (dtype) {
    case MG_F32: return ce_run_f32(dense, logits, labels, upstream, loss, dlogits, N, C, id64, s, rowloss_ext);
    case MG_F16: return ce_run_f16(dense, logits, labels, upstream, loss, dlogits, N, C, id64, s, rowloss_ext);
    default: return ce_run_bf16(dense, logits, labels, upstream, loss, dlogits, N, C, id64, s, rowloss_ext);
  }
}

static int ce_run_strided(const char* who, const void* logits, const void* labels, const void* upstream, void* loss,
                          void* dlogits, int rank, const int64_t* shape, const int64_t* la_strides,
                          const int64_t* lb_strides, int dtype, mg_stream stream) {
  if (rank < 1 || rank > kMaxRank) return fail(MG_ERR_INVALID, "%s: rank %d outside 1..%d", who, rank, kMaxRank);
  if (!shape || !la_strides || !lb_strides) return fail(MG_ERR_INVALID, "%s: null shape or strides", who);
  StridedView la{}, lb{};
  la.rank = lb.rank = rank;
  int64_t numel = 1;
  for (int d = 0; d < rank; ++d) {
    if (shape[d] <= 0) return fail(MG_ERR_INVALID, "%s: bad extent %lld in dim %d", who, static_cast<long long>(shape[d]), d);
    la.shape[d] = lb.shape[d] = shape[d];
    la.stride[d] = la_strides[d];
    lb.stride[d] = lb_strides[d];
    numel *= shape[d];
  }
  const int64_t C = shape[rank - 1];
  const int64_t N = numel / C;
  MG_TRY(check_ce(who, N, C, dtype));
  if (!logits || !labels || (!loss && !dlogits)) return fail(MG_ERR_INVALID, "%s: null pointer argument", who);
  hipStream_t s = to_stream(stream);
  switch (dtype) {
    case MG_F32: return ce_run_strided_f32(logits, labels, upstream, loss, dlogits, N, C, la, lb, s);
    case MG_F16: return ce_run_strided_f16(logits, labels, upstream, loss, dlogits, N, C, la, lb, s);
    default: return ce_run_strided_bf16(logits, labels, upstream, loss, dlogits, N, C, la, lb, s);
  }
}

// ---- The entry point that allocates nothing -------------------------------------------
// Per-row loss terms of mg_cross_entropy_fused_ids_noalloc live in this array instead of a
// pool block: MG_CE_NOALLOC_MAX_ROWS floats (4 MiB) on every GPU the library runs on, held
// until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; the device address it resolves to differs per GPU and is what the
// kernels receive.
static __device__ __align__(256) float scratch[MG_CE_NOALLOC_MAX_ROWS];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static float* g_scratch_ptr[kMaxDevices] = {};

// Resolves the current device's copy of `scratch` once; later calls return the kept address.
int ce_noalloc_setup(float** out) {
  int device = -1;
  MG_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices)
    return fail(MG_ERR_UNSUPPORTED, "cross_entropy_fused_ids_noalloc: device ordinal %d not supported", device);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    float* ptr = nullptr;
    MG_HIP(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
    if (ptr == nullptr) return fail(MG_ERR_HIP, "cross_entropy_fused_ids_noalloc: scratch symbol resolved to null");
    g_scratch_ptr[device] = ptr;
  }
  if (out) *out = g_scratch_ptr[device];
  return MG_OK;
}

}  // namespace mg

extern "C" {

int mg_cross_entropy(const void* logits, const void* labels, void* loss, int64_t N, int64_t C, int dtype,
                     mg_stream stream) {
  if (!loss) return mg::fail(MG_ERR_INVALID, "cross_entropy: null loss pointer");
  return mg::ce_run("cross_entropy", true, logits, labels, nullptr, loss, nullptr, N, C, dtype, 0, stream);
}

int mg_cross_entropy_grad(const void* logits, const void* labels, const void* upstream, void* dlogits, int64_t N,
                          int64_t C, int dtype, mg_stream stream) {
  if (!dlogits || !upstream) return mg::fail(MG_ERR_INVALID, "cross_entropy_grad: null pointer argument");
  return mg::ce_run("cross_entropy_grad", true, logits, labels, upstream, nullptr, dlogits, N, C, dtype, 0, stream);
}

int mg_cross_entropy_strided(const void* logits, const void* labels, void* loss, int rank, const int64_t* shape,
                             const int64_t* logits_strides, const int64_t* labels_strides, int dtype,
                             mg_stream stream) {
  if (!loss) return mg::fail(MG_ERR_INVALID, "cross_entropy_strided: null loss pointer");
  return mg::ce_run_strided("cross_entropy_strided", logits, labels, nullptr, loss, nullptr, rank, shape,
                            logits_strides, labels_strides, dtype, stream);
}

int mg_cross_entropy_grad_strided(const void* logits, const void* labels, const void* upstream, void* dlogits,
                                  int rank, const int64_t* shape, const int64_t* logits_strides,
                                  const int64_t* labels_strides, int dtype, mg_stream stream) {
  if (!dlogits || !upstream) return mg::fail(MG_ERR_INVALID, "cross_entropy_grad_strided: null pointer argument");
  return mg::ce_run_strided("cross_entropy_grad_strided", logits, labels, upstream, nullptr, dlogits, rank, shape,
                            logits_strides, labels_strides, dtype, stream);
}

int mg_cross_entropy_ids(const void* logits, const void* ids, void* loss, int64_t N, int64_t C, int dtype,
                         int id_dtype, mg_stream stream) {
  if (!loss) return mg::fail(MG_ERR_INVALID, "cross_entropy_ids: null loss pointer");
  return mg::ce_run("cross_entropy_ids", false, logits, ids, nullptr, loss, nullptr, N, C, dtype, id_dtype, stream);
}

int mg_cross_entropy_grad_ids(const void* logits, const void* ids, const void* upstream, void* dlogits, int64_t N,
                              int64_t C, int dtype, int id_dtype, mg_stream stream) {
  if (!dlogits) return mg::fail(MG_ERR_INVALID, "cross_entropy_grad_ids: null dlogits pointer");
  return mg::ce_run("cross_entropy_grad_ids", false, logits, ids, upstream, nullptr, dlogits, N, C, dtype, id_dtype,
                    stream);
}

int mg_cross_entropy_fused_ids(const void* logits, const void* ids, const void* upstream, void* loss, void* dlogits,
                               int64_t N, int64_t C, int dtype, int id_dtype, mg_stream stream) {
  if (!loss || !dlogits) return mg::fail(MG_ERR_INVALID, "cross_entropy_fused_ids: null output pointer");
  return mg::ce_run("cross_entropy_fused_ids", false, logits, ids, upstream, loss, dlogits, N, C, dtype, id_dtype,
                    stream);
}

int mg_cross_entropy_fused_ids_noalloc(const void* logits, const void* ids, const void* upstream, void* loss,
                                       void* dlogits, int64_t N, int64_t C, int dtype, int id_dtype,
                                       mg_stream stream) {
  if (!loss || !dlogits) return mg::fail(MG_ERR_INVALID, "cross_entropy_fused_ids_noalloc: null output pointer");
  if (N > MG_CE_NOALLOC_MAX_ROWS)
    return mg::fail(MG_ERR_INVALID, "cross_entropy_fused_ids_noalloc: N=%lld exceeds the %d rows of the static scratch",
                    static_cast<long long>(N), MG_CE_NOALLOC_MAX_ROWS);
  float* rowloss = nullptr;
  MG_TRY(mg::ce_noalloc_setup(&rowloss));
  return mg::ce_run("cross_entropy_fused_ids_noalloc", false, logits, ids, upstream, loss, dlogits, N, C, dtype,
                    id_dtype, stream, rowloss);
}

int mg_cross_entropy_fused(const void* logits, const void* labels, const void* upstream, void* loss, void* dlogits,
                           int64_t N, int64_t C, int dtype, mg_stream stream) {
  if (!loss || !dlogits) return mg::fail(MG_ERR_INVALID, "cross_entropy_fused: null output pointer");
  return mg::ce_run("cross_entropy_fused", true, logits, labels, upstream, loss, dlogits, N, C, dtype, 0, stream);
}

}  // extern "C"
