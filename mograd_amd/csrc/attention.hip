// C ABI for flash attention: argument checks, routing between the 16-bit MFMA kernels (16-bit
// storage, head dimension up to 256), the fp32 MFMA kernels (head dimension up to 128) and the
// general fp32 FMA kernels.
#include "attention_f32_mfma.h"
#include "attention_generic.h"
#include "attention_tiled.h"
#include "mg_internal.h"

namespace mg {

// attention_mfma.hip.  Return MG_ERR_UNSUPPORTED (without setting an error) when the
// shape is not one the MFMA kernels take.
bool attn_mfma_supported(int dtype, int64_t D, const void* const* ptrs, int nptrs);
int attn_fwd_mfma(const void* q, const void* k, const void* v, const void* mask, void* o, float* lse, AttnDims a,
                  float scale, bool causal, bool has_bias, int dtype, hipStream_t stream);
int attn_bwd_mfma(const void* d_o, const void* o, const void* q, const void* k, const void* v, const void* mask,
                  const float* lse, void* dq, void* dk, void* dv, AttnDims a, float scale, bool causal, bool has_bias,
                  int dtype, hipStream_t stream);

static int check_attn(const char* who, int64_t B, int64_t S, int64_t H, int64_t D, int causal, int has_bias, int dtype) {
  if (!is_float_dtype(dtype)) return fail(MG_ERR_INVALID, "%s: unsupported dtype %s", who, dtype_name(dtype));
  if (D <= 0 || D > 512) return fail(MG_ERR_INVALID, "%s: D=%lld out of range (1..512)", who, static_cast<long long>(D));
  if (causal != 0 && has_bias != 0)
    return fail(MG_ERR_INVALID, "%s: causal attention with additive bias is not supported", who);
  if (B <= 0 || S <= 0 || H <= 0 || B * H * S > 0x7fffffffLL || S > (1 << 24))
    return fail(MG_ERR_INVALID, "%s: bad shape B=%lld S=%lld H=%lld", who, static_cast<long long>(B),
                static_cast<long long>(S), static_cast<long long>(H));
  return MG_OK;
}

// The row-per-thread kernels (attention_tiled.h) take over once a sequence has rows for a
// workgroup; MOGRAD_HIP_ATTN_TILED=0 keeps the wave-per-row kernels.
static bool attn_tiled_ok(const AttnDims& a) {
  return a.D <= 512 && a.S >= 64 && static_cast<int64_t>(a.B) * a.H <= 65535 && env_int("MOGRAD_HIP_ATTN_TILED", 1) != 0;
}

// fp32 arithmetic on the matrix cores (attention_f32_mfma.h): head dims up to 128 once a sequence
// has rows for a workgroup; MOGRAD_HIP_ATTN_F32_MFMA=0 keeps the row-per-thread kernels.
static bool attn_f32_mfma_ok(const AttnDims& a) {
  return a.D <= kF32AttnMaxD && a.S >= 64 && ceil_div(a.S, kF32AttnBlock) <= 65535 &&
         env_int("MOGRAD_HIP_ATTN_F32_MFMA", 1) != 0;
}

template <typename T>
static void fwd_f32_mfma_launch(const void* q, const void* k, const void* v, const void* mask, void* o, float* lse,
                                const AttnDims& a, float scale, bool causal, bool has_bias, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(a.B * a.H), static_cast<unsigned>(ceil_div(a.S, kF32AttnBlock)));
#define MG_FWD_DP(DP_, C_, B_)                                                                                      \
  hipLaunchKernelGGL((attn_fwd_f32_mfma_kernel<T, DP_, C_, B_>), grid, dim3(256), 0, stream,                        \
                     static_cast<const T*>(q), static_cast<const T*>(k), static_cast<const T*>(v),                  \
                     static_cast<const T*>(mask), static_cast<T*>(o), lse, a, scale)
#define MG_FWD(C_, B_)                                                                                              \
  do {                                                                                                              \
    if (a.D <= 32) MG_FWD_DP(32, C_, B_);                                                                           \
    else if (a.D <= 64) MG_FWD_DP(64, C_, B_);                                                                      \
    else MG_FWD_DP(128, C_, B_);                                                                                    \
  } while (0)
  if (causal) MG_FWD(true, false);
  else if (has_bias) MG_FWD(false, true);
  else MG_FWD(false, false);
#undef MG_FWD
#undef MG_FWD_DP
}

template <typename T>
static void bwd_f32_mfma_launch(const void* d_o, const void* q, const void* k, const void* v, const void* mask,
                                const float* lse, const float* delta, void* dq, void* dk, void* dv, const AttnDims& a,
                                float scale, bool causal, bool has_bias, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(a.B * a.H), static_cast<unsigned>(ceil_div(a.S, kF32AttnBlock)));
#define MG_BWD_DP(DP_, C_, B_)                                                                                     \
  do {                                                                                                             \
    hipLaunchKernelGGL((attn_dkdv_f32_mfma_kernel<T, DP_, C_, B_>), grid, dim3(256), 0, stream,                    \
                       static_cast<const T*>(d_o), static_cast<const T*>(q), static_cast<const T*>(k),             \
                       static_cast<const T*>(v), static_cast<const T*>(mask), lse, delta, static_cast<T*>(dk),     \
                       static_cast<T*>(dv), a, scale);                                                             \
    hipLaunchKernelGGL((attn_dq_f32_mfma_kernel<T, DP_, C_, B_>), grid, dim3(256), 0, stream,                      \
                       static_cast<const T*>(d_o), static_cast<const T*>(q), static_cast<const T*>(k),             \
                       static_cast<const T*>(v), static_cast<const T*>(mask), lse, delta, static_cast<T*>(dq), a,  \
                       scale);                                                                                     \
  } while (0)
#define MG_BWD(C_, B_)                                                                                             \
  do {                                                                                                             \
    if (a.D <= 32) MG_BWD_DP(32, C_, B_);                                                                          \
    else if (a.D <= 64) MG_BWD_DP(64, C_, B_);                                                                     \
    else MG_BWD_DP(128, C_, B_);                                                                                   \
  } while (0)
  if (causal) MG_BWD(true, false);
  else if (has_bias) MG_BWD(false, true);
  else MG_BWD(false, false);
#undef MG_BWD
#undef MG_BWD_DP
}

template <typename T, int NT, int DL>
static void fwd_tiled_launch(const void* q, const void* k, const void* v, const void* mask, void* o, float* lse,
                             const AttnDims& a, float scale, bool causal, bool has_bias, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(ceil_div(a.S, 256 / NT)), static_cast<unsigned>(a.B * a.H));
#define MG_FWD(C_, B_)                                                                                               \
  hipLaunchKernelGGL((attn_fwd_tiled_kernel<T, NT, DL, C_, B_>), grid, dim3(256), 0, stream, static_cast<const T*>(q), \
                     static_cast<const T*>(k), static_cast<const T*>(v), static_cast<const T*>(mask),                \
                     static_cast<T*>(o), lse, a, scale)
  if (causal) MG_FWD(true, false);
  else if (has_bias) MG_FWD(false, true);
  else MG_FWD(false, false);
#undef MG_FWD
}

template <typename T, int NT, int DL, int NTK, int DLK>
static void bwd_tiled_launch(const void* d_o, const void* q, const void* k, const void* v, const void* mask,
                             const float* lse, const float* delta, void* dq, void* dk, void* dv, const AttnDims& a,
                             float scale, bool causal, bool has_bias, hipStream_t stream) {
  const dim3 grid_q(static_cast<unsigned>(ceil_div(a.S, 256 / NT)), static_cast<unsigned>(a.B * a.H));
  const dim3 grid_k(static_cast<unsigned>(ceil_div(a.S, 256 / NTK)), static_cast<unsigned>(a.B * a.H));
#define MG_BWD(C_, B_)                                                                                                \
  do {                                                                                                                \
    hipLaunchKernelGGL((attn_dq_tiled_kernel<T, NT, DL, C_, B_>), grid_q, dim3(256), 0, stream,                       \
                       static_cast<const T*>(d_o), static_cast<const T*>(q), static_cast<const T*>(k),                \
                       static_cast<const T*>(v), static_cast<const T*>(mask), lse, delta, static_cast<T*>(dq), a,     \
                       scale);                                                                                        \
    hipLaunchKernelGGL((attn_dkdv_tiled_kernel<T, NTK, DLK, C_, B_>), grid_k, dim3(256), 0, stream,                   \
                       static_cast<const T*>(d_o), static_cast<const T*>(q), static_cast<const T*>(k),                \
                       static_cast<const T*>(v), static_cast<const T*>(mask), lse, delta, static_cast<T*>(dk),        \
                       static_cast<T*>(dv), a, scale);                                                                \
  } while (0)
  if (causal) MG_BWD(true, false);
  else if (has_bias) MG_BWD(false, true);
  else MG_BWD(false, false);
#undef MG_BWD
}

template <typename T>
static int fwd_generic(const void* q, const void* k, const void* v, const void* mask, void* o, float* lse, AttnDims a,
                       float scale, bool causal, bool has_bias, hipStream_t stream) {
  const int64_t rows = static_cast<int64_t>(a.B) * a.H * a.S;
  if (attn_f32_mfma_ok(a)) {
    fwd_f32_mfma_launch<T>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }
  if (attn_tiled_ok(a)) {
    if (a.D <= 32) fwd_tiled_launch<T, 1, 32>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream);
    else if (a.D <= 64) fwd_tiled_launch<T, 2, 32>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream);
    else if (a.D <= 128) fwd_tiled_launch<T, 4, 32>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream);
    else if (a.D <= 256) fwd_tiled_launch<T, 8, 32>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream);
    else fwd_tiled_launch<T, 16, 32>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }
  const dim3 grid(static_cast<unsigned>(ceil_div(rows, 4)));
#define MG_FWD(C_, B_)                                                                                              \
  hipLaunchKernelGGL((attn_fwd_generic_kernel<T, C_, B_>), grid, dim3(256), 0, stream, static_cast<const T*>(q),    \
                     static_cast<const T*>(k), static_cast<const T*>(v), static_cast<const T*>(mask),               \
                     static_cast<T*>(o), lse, a, scale)
  if (causal) MG_FWD(true, false);
  else if (has_bias) MG_FWD(false, true);
  else MG_FWD(false, false);
#undef MG_FWD
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T>
static int bwd_generic(const void* d_o, const void* o, const void* q, const void* k, const void* v, const void* mask,
                       const float* lse, void* dq, void* dk, void* dv, AttnDims a, float scale, bool causal,
                       bool has_bias, hipStream_t stream) {
  const int64_t rows = static_cast<int64_t>(a.B) * a.H * a.S;
  Scratch delta;
  MG_TRY(delta.take(rows * static_cast<int64_t>(sizeof(float))));
  const dim3 grid(static_cast<unsigned>(ceil_div(rows, 4)));
  hipLaunchKernelGGL((attn_delta_kernel<T>), grid, dim3(256), 0, stream, static_cast<const T*>(d_o),
                     static_cast<const T*>(o), delta.as<float>(), rows, a.D, a.S, a.H, a.o_bshd);
  MG_LAUNCH_CHECK();
  if (attn_f32_mfma_ok(a)) {
    bwd_f32_mfma_launch<T>(d_o, q, k, v, mask, lse, delta.as<float>(), dq, dk, dv, a, scale, causal, has_bias, stream);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }
  if (attn_tiled_ok(a)) {
    const float* dl = delta.as<float>();
    if (a.D <= 32) bwd_tiled_launch<T, 1, 32, 1, 32>(d_o, q, k, v, mask, lse, dl, dq, dk, dv, a, scale, causal, has_bias, stream);
    else if (a.D <= 64) bwd_tiled_launch<T, 2, 32, 2, 32>(d_o, q, k, v, mask, lse, dl, dq, dk, dv, a, scale, causal, has_bias, stream);
    else if (a.D <= 128) bwd_tiled_launch<T, 4, 32, 4, 32>(d_o, q, k, v, mask, lse, dl, dq, dk, dv, a, scale, causal, has_bias, stream);
    else if (a.D <= 256) bwd_tiled_launch<T, 8, 32, 8, 32>(d_o, q, k, v, mask, lse, dl, dq, dk, dv, a, scale, causal, has_bias, stream);
    else bwd_tiled_launch<T, 16, 32, 16, 32>(d_o, q, k, v, mask, lse, dl, dq, dk, dv, a, scale, causal, has_bias, stream);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }
#define MG_BWD(C_, B_)                                                                                                \
  do {                                                                                                                \
    hipLaunchKernelGGL((attn_dq_generic_kernel<T, C_, B_>), grid, dim3(256), 0, stream, static_cast<const T*>(d_o),   \
                       static_cast<const T*>(q), static_cast<const T*>(k), static_cast<const T*>(v),                  \
                       static_cast<const T*>(mask), lse, delta.as<float>(), static_cast<T*>(dq), a, scale);           \
    hipLaunchKernelGGL((attn_dkdv_generic_kernel<T, C_, B_>), grid, dim3(256), 0, stream, static_cast<const T*>(d_o), \
                       static_cast<const T*>(q), static_cast<const T*>(k), static_cast<const T*>(v),                  \
                       static_cast<const T*>(mask), lse, delta.as<float>(), static_cast<T*>(dk), static_cast<T*>(dv), \
                       a, scale);                                                                                     \
  } while (0)
  if (causal) MG_BWD(true, false);
  else if (has_bias) MG_BWD(false, true);
  else MG_BWD(false, false);
#undef MG_BWD
  MG_LAUNCH_CHECK();
  return MG_OK;
}

}  // namespace mg

// o_bshd: O and dO are laid out (B, S, H, D) like Q, K, V instead of (B, H, S, D).
// ld: elements from one token's head-0 slice to the next token's in Q, K, V and their
// gradients; 0 means H * D (each tensor contiguous).
static int flash_attn_fwd_impl(int o_bshd, int64_t ld, const void* q, const void* k, const void* v, const void* mask,
                               void* o, float* lse, int64_t B, int64_t S, int64_t H, int64_t D, float scale, int causal,
                               int has_bias, int dtype, mg_stream stream) {
  MG_TRY(mg::check_attn("flash_attn_fwd", B, S, H, D, causal, has_bias, dtype));
  if (!q || !k || !v || !o || !lse || (has_bias && !mask))
    return mg::fail(MG_ERR_INVALID, "flash_attn_fwd: null pointer argument");
  const mg::AttnDims a{static_cast<int>(B), static_cast<int>(S), static_cast<int>(H), static_cast<int>(D),
                       o_bshd,              ld ? ld : H * D};
  hipStream_t s = mg::to_stream(stream);
  const void* ptrs[] = {q, k, v, o};  // the bias may start at any element
  if (mg::attn_mfma_supported(dtype, D, ptrs, 4))
    return mg::attn_fwd_mfma(q, k, v, mask, o, lse, a, scale, causal != 0, has_bias != 0, dtype, s);
  switch (dtype) {
    case MG_F32: return mg::fwd_generic<float>(q, k, v, mask, o, lse, a, scale, causal != 0, has_bias != 0, s);
    case MG_F16: return mg::fwd_generic<mg::f16_t>(q, k, v, mask, o, lse, a, scale, causal != 0, has_bias != 0, s);
    default: return mg::fwd_generic<mg::bf16_t>(q, k, v, mask, o, lse, a, scale, causal != 0, has_bias != 0, s);
  }
}

static int flash_attn_bwd_impl(int o_bshd, int64_t ld, const void* d_o, const void* o, const void* q, const void* k,
                               const void* v, const void* mask, const float* lse, void* dq, void* dk, void* dv,
                               int64_t B, int64_t S, int64_t H, int64_t D, float scale, int causal, int has_bias,
                               int dtype, mg_stream stream) {
  MG_TRY(mg::check_attn("flash_attn_bwd", B, S, H, D, causal, has_bias, dtype));
  if (!d_o || !o || !q || !k || !v || !lse || !dq || !dk || !dv || (has_bias && !mask))
    return mg::fail(MG_ERR_INVALID, "flash_attn_bwd: null pointer argument");
  const mg::AttnDims a{static_cast<int>(B), static_cast<int>(S), static_cast<int>(H), static_cast<int>(D),
                       o_bshd,              ld ? ld : H * D};
  hipStream_t s = mg::to_stream(stream);
  const void* ptrs[] = {d_o, o, q, k, v, dq, dk, dv};  // the bias may start at any element
  if (mg::attn_mfma_supported(dtype, D, ptrs, 8))
    return mg::attn_bwd_mfma(d_o, o, q, k, v, mask, lse, dq, dk, dv, a, scale, causal != 0, has_bias != 0, dtype, s);
  switch (dtype) {
    case MG_F32:
      return mg::bwd_generic<float>(d_o, o, q, k, v, mask, lse, dq, dk, dv, a, scale, causal != 0, has_bias != 0, s);
    case MG_F16:
      return mg::bwd_generic<mg::f16_t>(d_o, o, q, k, v, mask, lse, dq, dk, dv, a, scale, causal != 0, has_bias != 0, s);
    default:
      return mg::bwd_generic<mg::bf16_t>(d_o, o, q, k, v, mask, lse, dq, dk, dv, a, scale, causal != 0, has_bias != 0, s);
  }
}

extern "C" {

int mg_flash_attn_fwd(const void* q, const void* k, const void* v, const void* mask, void* o, float* lse, int64_t B,
                      int64_t S, int64_t H, int64_t D, float scale, int causal, int has_bias, int dtype,
                      mg_stream stream) {
  return flash_attn_fwd_impl(0, 0, q, k, v, mask, o, lse, B, S, H, D, scale, causal, has_bias, dtype, stream);
}

int mg_flash_attn_fwd_bshd(const void* q, const void* k, const void* v, const void* mask, void* o, float* lse, int64_t B,
                           int64_t S, int64_t H, int64_t D, float scale, int causal, int has_bias, int dtype,
                           mg_stream stream) {
  return flash_attn_fwd_impl(1, 0, q, k, v, mask, o, lse, B, S, H, D, scale, causal, has_bias, dtype, stream);
}

int mg_flash_attn_bwd(const void* d_o, const void* o, const void* q, const void* k, const void* v, const void* mask,
                      const float* lse, void* dq, void* dk, void* dv, int64_t B, int64_t S, int64_t H, int64_t D,
                      float scale, int causal, int has_bias, int dtype, mg_stream stream) {
  return flash_attn_bwd_impl(0, 0, d_o, o, q, k, v, mask, lse, dq, dk, dv, B, S, H, D, scale, causal, has_bias, dtype,
                             stream);
}

int mg_flash_attn_bwd_bshd(const void* d_o, const void* o, const void* q, const void* k, const void* v, const void* mask,
                           const float* lse, void* dq, void* dk, void* dv, int64_t B, int64_t S, int64_t H, int64_t D,
                           float scale, int causal, int has_bias, int dtype, mg_stream stream) {
  return flash_attn_bwd_impl(1, 0, d_o, o, q, k, v, mask, lse, dq, dk, dv, B, S, H, D, scale, causal, has_bias, dtype,
                             stream);
}

int mg_flash_attn_fwd_packed(const void* qkv, const void* mask, void* o, float* lse, int64_t B, int64_t S, int64_t H,
                             int64_t D, float scale, int causal, int has_bias, int dtype, mg_stream stream) {
  if (!qkv) return mg::fail(MG_ERR_INVALID, "flash_attn_fwd_packed: null pointer argument");
  const int64_t slice = H * D * mg::dtype_size(dtype);  // bytes from the Q slice of a token to its K slice
  const char* base = static_cast<const char*>(qkv);
  return flash_attn_fwd_impl(1, 3 * H * D, base, base + slice, base + 2 * slice, mask, o, lse, B, S, H, D, scale, causal,
                             has_bias, dtype, stream);
}

int mg_flash_attn_bwd_packed(const void* d_o, const void* o, const void* qkv, const void* mask, const float* lse,
                             void* dqkv, int64_t B, int64_t S, int64_t H, int64_t D, float scale, int causal,
                             int has_bias, int dtype, mg_stream stream) {
  if (!qkv || !dqkv) return mg::fail(MG_ERR_INVALID, "flash_attn_bwd_packed: null pointer argument");
  const int64_t slice = H * D * mg::dtype_size(dtype);
  const char* base = static_cast<const char*>(qkv);
  char* out = static_cast<char*>(dqkv);
  return flash_attn_bwd_impl(1, 3 * H * D, d_o, o, base, base + slice, base + 2 * slice, mask, lse, out, out + slice,
                             out + 2 * slice, B, S, H, D, scale, causal, has_bias, dtype, stream);
}

}  // extern "C"
