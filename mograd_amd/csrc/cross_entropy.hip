// C ABI for softmax cross-entropy: argument checks and dtype dispatch.
#include "mg_internal.h"

namespace mg {

#define MG_DECLARE_CROSS_ENTROPY(SUFFIX)                                                                         \
  int ce_run_##SUFFIX(bool, const void*, const void*, const void*, void*, void*, int64_t, int64_t, int,          \
                      hipStream_t);                                                                              \
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
                  void* dlogits, int64_t N, int64_t C, int dtype, int id_dtype, mg_stream stream) {
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
    case MG_F32: return ce_run_f32(dense, logits, labels, upstream, loss, dlogits, N, C, id64, s);
    case MG_F16: return ce_run_f16(dense, logits, labels, upstream, loss, dlogits, N, C, id64, s);
    default: return ce_run_bf16(dense, logits, labels, upstream, loss, dlogits, N, C, id64, s);
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

int mg_cross_entropy_fused(const void* logits, const void* labels, const void* upstream, void* loss, void* dlogits,
                           int64_t N, int64_t C, int dtype, mg_stream stream) {
  if (!loss || !dlogits) return mg::fail(MG_ERR_INVALID, "cross_entropy_fused: null output pointer");
  return mg::ce_run("cross_entropy_fused", true, logits, labels, upstream, loss, dlogits, N, C, dtype, 0, stream);
}

}  // extern "C"
