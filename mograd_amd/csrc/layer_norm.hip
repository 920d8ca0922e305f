// C ABI for LayerNorm: argument checks and dtype dispatch.
#include "mg_deferred.h"
#include "mg_internal.h"

namespace mg {
#define MG_DECLARE_LAYER_NORM(SUFFIX)                                                                         \
  int ln_fwd_##SUFFIX(const void*, const void*, const void*, void*, float*, float*, int64_t, int64_t, float,  \
                      hipStream_t);                                                                           \
  int ln_bwd_##SUFFIX(const void*, const void*, const void*, const float*, const float*, const void*, void*,  \
                      void*, void*, int64_t, int64_t, float, int, hipStream_t);
MG_DECLARE_LAYER_NORM(f32)
MG_DECLARE_LAYER_NORM(f16)
MG_DECLARE_LAYER_NORM(bf16)
#undef MG_DECLARE_LAYER_NORM

static int check_ln(const char* who, int64_t rows, int64_t cols, int dtype) {
  if (!is_float_dtype(dtype)) return fail(MG_ERR_INVALID, "%s: unsupported dtype %s", who, dtype_name(dtype));
  if (rows < 0 || cols <= 0 || cols > 0x3fffffffLL || rows > 0x7fffffffLL)
    return fail(MG_ERR_INVALID, "%s: bad shape rows=%lld cols=%lld", who, static_cast<long long>(rows),
                static_cast<long long>(cols));
  return MG_OK;
}

static int ln_fwd(const void* x, const void* gamma, const void* beta, void* y, float* mean, float* rstd, int64_t rows,
                  int64_t cols, float eps, int dtype, mg_stream stream) {
  MG_TRY(check_ln("layer_norm_fwd", rows, cols, dtype));
  if (rows == 0) return MG_OK;
  if (!x || !gamma || !beta || !y) return fail(MG_ERR_INVALID, "layer_norm_fwd: null pointer argument");
  hipStream_t s = to_stream(stream);
  switch (dtype) {
    case MG_F32: return ln_fwd_f32(x, gamma, beta, y, mean, rstd, rows, cols, eps, s);
    case MG_F16: return ln_fwd_f16(x, gamma, beta, y, mean, rstd, rows, cols, eps, s);
    default: return ln_fwd_bf16(x, gamma, beta, y, mean, rstd, rows, cols, eps, s);
  }
}

// (also the second half of mg_linear_bwd_layer_norm_bwd when its shapes take separate kernels)
int ln_bwd(const void* dy, const void* x, const void* gamma, const float* mean, const float* rstd,
           const void* residual, void* dx, void* dgamma, void* dbeta, int64_t rows, int64_t cols, float eps,
                  int dtype, mg_stream stream) {
  MG_TRY(check_ln("layer_norm_bwd", rows, cols, dtype));
  if (!dgamma || !dbeta) return fail(MG_ERR_INVALID, "layer_norm_bwd: null pointer argument");
  hipStream_t s = to_stream(stream);
  if (rows == 0) {  // the column sums of an empty matrix are zero
    // zero fill by kernel, not hipMemsetAsync: safe to record into a HIP graph
    MG_TRY(mg_fill(dgamma, 0.0, cols, dtype, s));
    MG_TRY(mg_fill(dbeta, 0.0, cols, dtype, s));
    return MG_OK;
  }
  if (!dy || !x || !gamma || !dx) return fail(MG_ERR_INVALID, "layer_norm_bwd: null pointer argument");
  switch (dtype) {
    case MG_F32: return ln_bwd_f32(dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta, rows, cols, eps, dtype, s);
    case MG_F16: return ln_bwd_f16(dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta, rows, cols, eps, dtype, s);
    default: return ln_bwd_bf16(dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta, rows, cols, eps, dtype, s);
  }
}

}  // namespace mg

extern "C" {

int mg_layer_norm_fwd(const void* x, const void* gamma, const void* beta, void* y, int64_t rows, int64_t cols,
                      float eps, int dtype, mg_stream stream) {
  return mg::ln_fwd(x, gamma, beta, y, nullptr, nullptr, rows, cols, eps, dtype, stream);
}

int mg_layer_norm_fwd_stats(const void* x, const void* gamma, const void* beta, void* y, float* mean, float* rstd,
                            int64_t rows, int64_t cols, float eps, int dtype, mg_stream stream) {
  if (!mean || !rstd) return mg::fail(MG_ERR_INVALID, "layer_norm_fwd_stats: null statistics pointer");
  return mg::ln_fwd(x, gamma, beta, y, mean, rstd, rows, cols, eps, dtype, stream);
}

int mg_layer_norm_bwd(const void* dy, const void* x, const void* gamma, void* dx, void* dgamma, void* dbeta,
                      int64_t rows, int64_t cols, float eps, int dtype, mg_stream stream) {
  return mg::ln_bwd(dy, x, gamma, nullptr, nullptr, nullptr, dx, dgamma, dbeta, rows, cols, eps, dtype, stream);
}

int mg_layer_norm_bwd_stats(const void* dy, const void* x, const void* gamma, const float* mean, const float* rstd,
                            void* dx, void* dgamma, void* dbeta, int64_t rows, int64_t cols, int dtype,
                            mg_stream stream) {
  if (!mean || !rstd) return mg::fail(MG_ERR_INVALID, "layer_norm_bwd_stats: null statistics pointer");
  return mg::ln_bwd(dy, x, gamma, mean, rstd, nullptr, dx, dgamma, dbeta, rows, cols, 0.f, dtype, stream);
}

int mg_layer_norm_bwd_stats_add(const void* dy, const void* x, const void* gamma, const float* mean, const float* rstd,
                                const void* residual, void* dx, void* dgamma, void* dbeta, int64_t rows, int64_t cols,
                                int dtype, mg_stream stream) {
  if (!mean || !rstd) return mg::fail(MG_ERR_INVALID, "layer_norm_bwd_stats_add: null statistics pointer");
  if (!residual && rows > 0) return mg::fail(MG_ERR_INVALID, "layer_norm_bwd_stats_add: null residual pointer");
  return mg::ln_bwd(dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta, rows, cols, 0.f, dtype, stream);
}

int mg_layer_norm_bwd_stats_deferred(const void* dy, const void* x, const void* gamma, const float* mean,
                                     const float* rstd, const void* residual, void* dx, void* dgamma, void* dbeta,
                                     int64_t rows, int64_t cols, int dtype, int grad_dtype, mg_deferred list,
                                     mg_stream stream) {
  if (!mean || !rstd) return mg::fail(MG_ERR_INVALID, "layer_norm_bwd_stats_deferred: null statistics pointer");
  MG_TRY(mg::check_ln("layer_norm_bwd_stats_deferred", rows, cols, dtype));
  MG_TRY(mg::deferred_check("layer_norm_bwd_stats_deferred", list, dtype, grad_dtype));
  if (!dgamma || !dbeta) return mg::fail(MG_ERR_INVALID, "layer_norm_bwd_stats_deferred: null pointer argument");
  mg::DeferredScope scope(static_cast<mg::DeferredList*>(list), dtype, grad_dtype);
  void *dg_use, *db_use;
  MG_TRY(scope.substitute(dgamma, cols, &dg_use));
  MG_TRY(scope.substitute(dbeta, cols, &db_use));
  MG_TRY(mg::ln_bwd(dy, x, gamma, mean, rstd, residual, dx, dg_use, db_use, rows, cols, 0.f, dtype, stream));
  return scope.finish(mg::to_stream(stream));
}

}  // extern "C"
