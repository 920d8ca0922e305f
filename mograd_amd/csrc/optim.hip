// Optimizer updates as single streaming kernels over flat fp32 arrays: Adam / AdamW and
// SGD.  The reference builds each update from a chain of elementwise ops
// (mograd/nn/optim/adam.mojo:6-78, sgd.mojo:24-45); the arithmetic and its order are the
// same here, in one pass: 28 bytes moved per parameter for Adam, 12 for SGD.
#include "mg_device.h"
#include <cmath>

#include "mg_internal.h"

// No fused multiply-add contraction in this file: each operation of an update is rounded
// on its own, in the order the reference's chain of elementwise kernels applies them, so an
// fp32 emulation of that chain gives the same bits.
#pragma clang fp contract(off)

namespace mg {

struct AdamParams {
  float lr, beta1, beta2, eps, weight_decay;
  float one_minus_beta1, one_minus_beta2;
  float inv_bc1, inv_bc2;  // 1 / (1 - beta^t)
  float decay;             // 1 - lr * weight_decay
  int decoupled;
};

// Plain operators: compiled under the pragma above they carry no permission to contract
// (the header's __fmul_rn/__fadd_rn wrappers are compiled without it and would fuse).
__device__ __forceinline__ float mul_rn(float a, float b) { return a * b; }
__device__ __forceinline__ float add_rn(float a, float b) { return a + b; }
__device__ __forceinline__ float sub_rn(float a, float b) { return a - b; }

__device__ __forceinline__ void adam_one(float& w, float g, float& m, float& v, const AdamParams& p) {
  if (!p.decoupled && p.weight_decay > 0.f) g = add_rn(g, mul_rn(w, p.weight_decay));
  m = add_rn(mul_rn(m, p.beta1), mul_rn(g, p.one_minus_beta1));
  v = add_rn(mul_rn(v, p.beta2), mul_rn(mul_rn(g, g), p.one_minus_beta2));
  const float m_hat = mul_rn(m, p.inv_bc1);
  const float v_hat = mul_rn(v, p.inv_bc2);
  const float update = mul_rn(__fdiv_rn(m_hat, add_rn(__fsqrt_rn(v_hat), p.eps)), p.lr);
  const float base = (p.decoupled && p.weight_decay > 0.f) ? mul_rn(w, p.decay) : w;
  w = sub_rn(base, update);
}

__global__ __launch_bounds__(256) void adam_kernel(float* __restrict__ w, const float* __restrict__ g,
                                                   float* __restrict__ m, float* __restrict__ v, int64_t n,
                                                   AdamParams p) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * 4;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4; i < n; i += stride) {
    if (i + 4 <= n) {
      float4 w4 = *reinterpret_cast<const float4*>(w + i);
      const float4 g4 = *reinterpret_cast<const float4*>(g + i);
      float4 m4 = *reinterpret_cast<const float4*>(m + i);
      float4 v4 = *reinterpret_cast<const float4*>(v + i);
      adam_one(w4.x, g4.x, m4.x, v4.x, p);
      adam_one(w4.y, g4.y, m4.y, v4.y, p);
      adam_one(w4.z, g4.z, m4.z, v4.z, p);
      adam_one(w4.w, g4.w, m4.w, v4.w, p);
      *reinterpret_cast<float4*>(w + i) = w4;
      *reinterpret_cast<float4*>(m + i) = m4;
      *reinterpret_cast<float4*>(v + i) = v4;
    } else {
      for (int64_t j = i; j < n; ++j) adam_one(w[j], g[j], m[j], v[j], p);
    }
  }
}

__global__ __launch_bounds__(256) void sgd_kernel(float* __restrict__ w, const float* __restrict__ g, int64_t n,
                                                  float lr) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * 4;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4; i < n; i += stride) {
    if (i + 4 <= n) {
      float4 w4 = *reinterpret_cast<const float4*>(w + i);
      const float4 g4 = *reinterpret_cast<const float4*>(g + i);
      w4.x = sub_rn(w4.x, mul_rn(g4.x, lr));
      w4.y = sub_rn(w4.y, mul_rn(g4.y, lr));
      w4.z = sub_rn(w4.z, mul_rn(g4.z, lr));
      w4.w = sub_rn(w4.w, mul_rn(g4.w, lr));
      *reinterpret_cast<float4*>(w + i) = w4;
    } else {
      for (int64_t j = i; j < n; ++j) w[j] = sub_rn(w[j], mul_rn(g[j], lr));
    }
  }
}

static unsigned optim_blocks(int64_t n) {
  int64_t blocks = ceil_div(n, 1024);
  const int64_t cap = static_cast<int64_t>(device_info().cu_count) * 16;
  if (blocks > cap) blocks = cap;
  return static_cast<unsigned>(blocks < 1 ? 1 : blocks);
}

}  // namespace mg

extern "C" {

int mg_adam_step(void* w, const void* g, void* m, void* v, int64_t n, float lr, float beta1, float beta2, float eps,
                 float weight_decay, int64_t t, int decoupled_weight_decay, mg_stream stream) {
  if (n < 0) return mg::fail(MG_ERR_INVALID, "adam_step: negative size");
  if (t < 1) return mg::fail(MG_ERR_INVALID, "adam_step: step count t=%lld must be >= 1", static_cast<long long>(t));
  if (n == 0) return MG_OK;
  if (!w || !g || !m || !v) return mg::fail(MG_ERR_INVALID, "adam_step: null pointer argument");
  if (!mg::aligned16(w) || !mg::aligned16(g) || !mg::aligned16(m) || !mg::aligned16(v))
    return mg::fail(MG_ERR_INVALID, "adam_step: pointers must be 16-byte aligned");
  // Bias corrections `Float32(1.0) - beta**t` (mograd/nn/optim/adam.mojo:19-20).  The power is
  // taken in double and rounded to fp32 once: constant time in t, and within one fp32 rounding
  // of the exact value however large the step count (a chain of t fp32 multiplications costs
  // O(t) host time per call and drifts by up to t/2 ulp).
  const float b1t = static_cast<float>(std::pow(static_cast<double>(beta1), static_cast<double>(t)));
  const float b2t = static_cast<float>(std::pow(static_cast<double>(beta2), static_cast<double>(t)));
  mg::AdamParams p{lr,
                   beta1,
                   beta2,
                   eps,
                   weight_decay,
                   1.0f - beta1,
                   1.0f - beta2,
                   1.0f / (1.0f - b1t),
                   1.0f / (1.0f - b2t),
                   1.0f - lr * weight_decay,
                   decoupled_weight_decay != 0};
  hipLaunchKernelGGL(mg::adam_kernel, dim3(mg::optim_blocks(n)), dim3(256), 0, mg::to_stream(stream),
                     static_cast<float*>(w), static_cast<const float*>(g), static_cast<float*>(m), static_cast<float*>(v),
                     n, p);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

int mg_sgd_step(void* w, const void* g, int64_t n, float lr, mg_stream stream) {
  if (n < 0) return mg::fail(MG_ERR_INVALID, "sgd_step: negative size");
  if (n == 0) return MG_OK;
  if (!w || !g) return mg::fail(MG_ERR_INVALID, "sgd_step: null pointer argument");
  if (!mg::aligned16(w) || !mg::aligned16(g)) return mg::fail(MG_ERR_INVALID, "sgd_step: pointers must be 16-byte aligned");
  hipLaunchKernelGGL(mg::sgd_kernel, dim3(mg::optim_blocks(n)), dim3(256), 0, mg::to_stream(stream),
                     static_cast<float*>(w), static_cast<const float*>(g), n, lr);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

}  // extern "C"
