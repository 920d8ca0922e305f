// Device-side helpers for gfx950 (wave64): storage types, 128-bit vector access,
// DPP wave reductions and workgroup reductions.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mg {

constexpr int kWave = 64;

// ------------------------------------------------------------------------------------
// Storage element types.  All arithmetic is fp32; these only describe memory.
// ------------------------------------------------------------------------------------

struct bf16_t {
  uint16_t bits;
};
using f16_t = _Float16;

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(f16_t v) { return static_cast<float>(v); }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(static_cast<uint32_t>(v.bits) << 16); }

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ f16_t from_float<f16_t>(float v) {
  return static_cast<f16_t>(v);
}
// fp32 -> bf16, round to nearest even, NaN stays NaN: the hardware conversion
// (v_cvt_pk_bf16_f32, one instruction for two values; the bit arithmetic it replaces took
// seven per value, which showed in every 16-bit kernel's output loop).
typedef __bf16 hw_bf16x2 __attribute__((ext_vector_type(2)));
typedef float hw_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf16_pack2_rne(float lo, float hi) {
  const hw_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, hw_bf16x2));
}
__device__ __forceinline__ uint16_t bf16_bits_rne(float v) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
  return bf16_t{bf16_bits_rne(v)};
}

// ------------------------------------------------------------------------------------
// Vector access: VEC consecutive elements of T as fp32 values.  With VEC * sizeof(T)
// == 16 this is one 128-bit load/store; the address must then be 16-byte aligned.
// ------------------------------------------------------------------------------------

template <typename T, int VEC>
struct VecIO;

// `load_stream` reads past the caches (a non-temporal load): for inputs larger than the caches that a
// kernel reads once and writes nothing of comparable size next to (the cross-entropy loss over
// 1.65 GB of logits 266 -> 238 us, 6.9 TB/s).  A kernel that writes as much as it reads gains nothing
// from it, and on an input that is still cached it is the slower load (a 33 MB column sum 6.3 -> 11 us).
// `store_stream` writes past the caches (a non-temporal store): for outputs that are written
// once and read by a later kernel.  On buffers that are not cache-resident it is the faster form
// for the row and elementwise kernels (LayerNorm backward (2048, 4096) fp32: 33.9 -> 28.8 us, a
// 100 MB add 19.9 -> 15.6 us; no difference on cache-resident ones), but not for the
// cross-entropy kernels, whose workgroups write a long row each (631 -> 889 us at (8192, 50304)),
// and they keep the plain store.
typedef float mg_f4 __attribute__((ext_vector_type(4)));
typedef uint32_t mg_u4 __attribute__((ext_vector_type(4)));

template <>
struct VecIO<float, 4> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    float4 r = *reinterpret_cast<const float4*>(p);
    v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
  }
  static __device__ __forceinline__ void load_stream(const float* p, float (&v)[4]) {
    const mg_f4 r = __builtin_nontemporal_load(reinterpret_cast<const mg_f4*>(p));
    v[0] = r[0]; v[1] = r[1]; v[2] = r[2]; v[3] = r[3];
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
  static __device__ __forceinline__ void store_stream(float* p, const float (&v)[4]) {
    const mg_f4 r = {v[0], v[1], v[2], v[3]};
    __builtin_nontemporal_store(r, reinterpret_cast<mg_f4*>(p));
  }
};

template <typename T>
struct VecIO<T, 1> {
  static __device__ __forceinline__ void load(const T* p, float (&v)[1]) { v[0] = to_float(*p); }
  static __device__ __forceinline__ void load_stream(const T* p, float (&v)[1]) { v[0] = to_float(*p); }
  static __device__ __forceinline__ void store(T* p, const float (&v)[1]) { *p = from_float<T>(v[0]); }
  static __device__ __forceinline__ void store_stream(T* p, const float (&v)[1]) { *p = from_float<T>(v[0]); }
};

template <>
struct VecIO<f16_t, 8> {
  static __device__ __forceinline__ void unpack(const uint32_t (&w)[4], float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      union { uint32_t u; f16_t h[2]; } cv;
      cv.u = w[i];
      v[2 * i] = static_cast<float>(cv.h[0]);
      v[2 * i + 1] = static_cast<float>(cv.h[1]);
    }
  }
  static __device__ __forceinline__ void load(const f16_t* p, float (&v)[8]) {
    uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
    unpack(w, v);
  }
  static __device__ __forceinline__ void load_stream(const f16_t* p, float (&v)[8]) {
    const mg_u4 r = __builtin_nontemporal_load(reinterpret_cast<const mg_u4*>(p));
    const uint32_t w[4] = {r[0], r[1], r[2], r[3]};
    unpack(w, v);
  }
  static __device__ __forceinline__ void store(f16_t* p, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      union { uint32_t u; f16_t h[2]; } cv;
      cv.h[0] = static_cast<f16_t>(v[2 * i]);
      cv.h[1] = static_cast<f16_t>(v[2 * i + 1]);
      w[i] = cv.u;
    }
    *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
  }
  static __device__ __forceinline__ void store_stream(f16_t* p, const float (&v)[8]) {
    mg_u4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      union { uint32_t u; f16_t h[2]; } cv;
      cv.h[0] = static_cast<f16_t>(v[2 * i]);
      cv.h[1] = static_cast<f16_t>(v[2 * i + 1]);
      w[i] = cv.u;
    }
    __builtin_nontemporal_store(w, reinterpret_cast<mg_u4*>(p));
  }
};

template <>
struct VecIO<bf16_t, 8> {
  static __device__ __forceinline__ void unpack(const uint32_t (&w)[4], float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
    unpack(w, v);
  }
  static __device__ __forceinline__ void load_stream(const bf16_t* p, float (&v)[8]) {
    const mg_u4 r = __builtin_nontemporal_load(reinterpret_cast<const mg_u4*>(p));
    const uint32_t w[4] = {r[0], r[1], r[2], r[3]};
    unpack(w, v);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = bf16_pack2_rne(v[2 * i], v[2 * i + 1]);
    *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
  }
  static __device__ __forceinline__ void store_stream(bf16_t* p, const float (&v)[8]) {
    mg_u4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = bf16_pack2_rne(v[2 * i], v[2 * i + 1]);
    __builtin_nontemporal_store(w, reinterpret_cast<mg_u4*>(p));
  }
};

// Widest vector this library uses for T: 16 bytes.
template <typename T>
struct WideVec {
  static constexpr int value = 16 / static_cast<int>(sizeof(T));
};

// ------------------------------------------------------------------------------------
// Wave reductions with DPP (no LDS traffic for the first four steps).
// ------------------------------------------------------------------------------------

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

constexpr int kDppQuadXor1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;
constexpr int kSwizzleXor16 = 0x401F;   // ds_swizzle bit mode: and 0x1f, or 0, xor 0x10

struct SumOp {
  static __device__ __forceinline__ float apply(float a, float b) { return a + b; }
};
struct MaxOp {
  static __device__ __forceinline__ float apply(float a, float b) { return fmaxf(a, b); }
};

// Every lane returns the reduction over all 64 lanes.
template <typename Op>
__device__ __forceinline__ float wave_allreduce(float v) {
  v = Op::apply(v, dpp_move<kDppQuadXor1>(v));
  v = Op::apply(v, dpp_move<kDppQuadXor2>(v));
  v = Op::apply(v, dpp_move<kDppRowHalfMirror>(v));
  v = Op::apply(v, dpp_move<kDppRowMirror>(v));
  v = Op::apply(v, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), kSwizzleXor16)));
  float lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  return Op::apply(lo, hi);
}

// Every lane returns the reduction over its own row of 16 lanes (lanes 16j .. 16j+15): the
// first four DPP steps of wave_allreduce, which never leave a row.
template <typename Op>
__device__ __forceinline__ float row16_allreduce(float v) {
  v = Op::apply(v, dpp_move<kDppQuadXor1>(v));
  v = Op::apply(v, dpp_move<kDppQuadXor2>(v));
  v = Op::apply(v, dpp_move<kDppRowHalfMirror>(v));
  v = Op::apply(v, dpp_move<kDppRowMirror>(v));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) { return wave_allreduce<SumOp>(v); }
__device__ __forceinline__ float wave_max(float v) { return wave_allreduce<MaxOp>(v); }

// ------------------------------------------------------------------------------------
// Workgroup reductions over NW waves.  `slots` is LDS of at least 2 * K * NW floats; the
// caller alternates `phase` (0/1) between consecutive reductions so that one barrier per
// reduction is enough: a wave can only overwrite a slot two reductions later, after the
// intervening barrier.
// ------------------------------------------------------------------------------------

template <typename Op, int NW, int K>
__device__ __forceinline__ void block_allreduce(float (&v)[K], float* slots, int phase) {
#pragma unroll
  for (int k = 0; k < K; ++k) v[k] = wave_allreduce<Op>(v[k]);
  if constexpr (NW == 1) return;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  float* base = slots + phase * (K * NW);
  if (lane == 0) {
#pragma unroll
    for (int k = 0; k < K; ++k) base[k * NW + wave] = v[k];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < K; ++k) {
    float acc = base[k * NW];
#pragma unroll
    for (int w = 1; w < NW; ++w) acc = Op::apply(acc, base[k * NW + w]);
    v[k] = acc;
  }
}

// The same over groups of GW consecutive waves (a row shared by part of the workgroup): every
// wave publishes its sums, one barrier for the whole workgroup, every thread adds up the GW
// slots of its own group.  All waves of the workgroup must call it together.
template <typename Op, int NW, int GW, int K>
__device__ __forceinline__ void group_allreduce(float (&v)[K], float* slots, int phase) {
  static_assert(NW % GW == 0, "whole groups");
#pragma unroll
  for (int k = 0; k < K; ++k) v[k] = wave_allreduce<Op>(v[k]);
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  float* base = slots + phase * (K * NW);
  if (lane == 0) {
#pragma unroll
    for (int k = 0; k < K; ++k) base[k * NW + wave] = v[k];
  }
  __syncthreads();
  const int first = wave / GW * GW;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    float acc = base[k * NW + first];
#pragma unroll
    for (int w = 1; w < GW; ++w) acc = Op::apply(acc, base[k * NW + first + w]);
    v[k] = acc;
  }
}

}  // namespace mg
