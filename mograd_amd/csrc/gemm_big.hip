// Launches of gemm_16bit_big_kernel (256 x 256 output tiles, four waves of 128 x 128), in a
// translation unit of their own so that they compile beside the other GEMM kernels.
#include "gemm_impl.h"

namespace mg {

template <typename T, bool A_KC, bool B_KC>
static int big_launch_typed(int variant, const void* a_, const void* b_, const void* bias_, void* c_, int64_t batch,
                            int M, int N, int K, int64_t lda, int64_t ldb, int64_t bsa, int64_t bsb,
                            const void* residual, const void* relu_mask, int relu, hipStream_t stream) {
  const T* a = static_cast<const T*>(a_);
  const T* b = static_cast<const T*>(b_);
  const T* bias = static_cast<const T*>(bias_);
  T* c = static_cast<T*>(c_);
  const int tiles_m = static_cast<int>(ceil_div(M, kGemmBigT)), tiles_n = static_cast<int>(ceil_div(N, kGemmBigT));
  const int64_t blocks = static_cast<int64_t>(tiles_m) * tiles_n * batch;
  if (blocks > 0x7fffffffLL) return fail(MG_ERR_INVALID, "matmul: too many output tiles");
  const GemmEpilogue<T> ep{static_cast<const T*>(residual), static_cast<const T*>(relu_mask), relu};
  const int64_t ldc = N, bsc = static_cast<int64_t>(M) * N;
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, a, b, bias, c, M, N, K, lda, ldb,
                       ldc, bsa, bsb, bsc, tiles_m, tiles_n, ep);
  };
  auto pick = [&](auto has_bias) {
    constexpr bool HB = decltype(has_bias)::value;
    if (variant == 4324) launch(gemm_16bit_big_kernel<T, A_KC, B_KC, HB, 32, 4>);
    else launch(gemm_16bit_big_kernel<T, A_KC, B_KC, HB, 64, 2>);
  };
  if (bias) pick(std::true_type{});
  else pick(std::false_type{});
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T>
static int big_launch_layout(bool a_kc, bool b_kc, int variant, const void* a, const void* b, const void* bias, void* c,
                             int64_t batch, int M, int N, int K, int64_t lda, int64_t ldb, int64_t bsa, int64_t bsb,
                             const void* residual, const void* relu_mask, int relu, hipStream_t stream) {
#define MG_BIG(AK, BK_) \
  big_launch_typed<T, AK, BK_>(variant, a, b, bias, c, batch, M, N, K, lda, ldb, bsa, bsb, residual, relu_mask, relu, stream)
  if (a_kc && b_kc) return MG_BIG(true, true);
  if (a_kc) return MG_BIG(true, false);
  if (b_kc) return MG_BIG(false, true);
  return MG_BIG(false, false);
#undef MG_BIG
}

int gemm16_big_launch(int dtype, bool a_kc, bool b_kc, int variant, const void* a, const void* b, const void* bias,
                      void* c, int64_t batch, int M, int N, int K, int64_t lda, int64_t ldb, int64_t bsa, int64_t bsb,
                      const void* residual, const void* relu_mask, int relu, hipStream_t stream) {
  if (dtype == MG_BF16)
    return big_launch_layout<bf16_t>(a_kc, b_kc, variant, a, b, bias, c, batch, M, N, K, lda, ldb, bsa, bsb, residual,
                                     relu_mask, relu, stream);
  return big_launch_layout<f16_t>(a_kc, b_kc, variant, a, b, bias, c, batch, M, N, K, lda, ldb, bsa, bsb, residual,
                                  relu_mask, relu, stream);
}

}  // namespace mg
