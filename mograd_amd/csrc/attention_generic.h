// Flash attention, general path: any of the three float types, any head dimension up to
// 512, additive bias or causal masking.  fp32 arithmetic throughout, one wave per row,
// nothing of size S x S is stored.  This is the path for fp32 tensors (where it meets the
// fp32 error budget) and for shapes the MFMA kernels do not cover.
//
// Layouts: Q, K, V, dQ, dK, dV are BSHD; O and dO are BHSD; mask is (B, H, S, S); LSE and
// delta are (B, H, S) fp32, LSE in natural-log units.
#pragma once

#include "mg_device.h"
#include "mg_internal.h"

namespace mg {

constexpr float kAttnLog2e = 1.4426950408889634f;
constexpr float kAttnLn2 = 0.6931471805599453f;
constexpr int kAttnMaxDPerLane = 8;  // 512 / 64

struct AttnDims {
  int B, S, H, D;
  // O and dO are (B,H,S,D) in the reference's contract; with o_bshd they are (B,S,H,D) like
  // Q, K and V, which is what a projection that follows (or precedes) attention reads.
  int o_bshd = 0;
  // Elements between consecutive tokens of Q, K, V (and dQ, dK, dV): H*D when each is its
  // own (B,S,H,D) tensor, 3*H*D when they are the three slices of one (B,S,3,H,D) tensor.
  int64_t ld = 0;
};

__device__ __forceinline__ int64_t bshd(const AttnDims& a, int b, int s, int h) {
  return ((static_cast<int64_t>(b) * a.S + s) * a.H + h) * a.D;
}
__device__ __forceinline__ int64_t bhsd(const AttnDims& a, int b, int h, int s) {
  return ((static_cast<int64_t>(b) * a.H + h) * a.S + s) * a.D;
}
// Offset of row (b, s, h) of Q, K, V, dQ, dK or dV.
__device__ __forceinline__ int64_t qkv_at(const AttnDims& a, int b, int s, int h) {
  return (static_cast<int64_t>(b) * a.S + s) * a.ld + static_cast<int64_t>(h) * a.D;
}
// Offset of row (b, h, s) of O / dO, and the distance between consecutive s of one (b, h).
__device__ __forceinline__ int64_t o_at(const AttnDims& a, int b, int h, int s) {
  return a.o_bshd ? bshd(a, b, s, h) : bhsd(a, b, h, s);
}
__device__ __forceinline__ int64_t o_ld(const AttnDims& a) { return a.o_bshd ? static_cast<int64_t>(a.H) * a.D : a.D; }
// delta and LSE are always (B,H,S): index of the statistics of row `row` of O in O's own row order.
__device__ __forceinline__ int64_t o_row_to_bhs(int64_t row, int S, int H, int o_bshd) {
  if (!o_bshd) return row;
  const int64_t h = row % H, bs = row / H;
  return ((bs / S) * H + h) * S + bs % S;
}

// A row of D elements spread over the 64 lanes: lane l holds d = l, l + 64, ...
template <typename T>
__device__ __forceinline__ void load_row(const T* __restrict__ p, int D, int lane, float (&v)[kAttnMaxDPerLane]) {
#pragma unroll
  for (int i = 0; i < kAttnMaxDPerLane; ++i) {
    const int d = lane + i * kWave;
    v[i] = d < D ? to_float(p[d]) : 0.f;
  }
}

__device__ __forceinline__ float dot_rows(const float (&a)[kAttnMaxDPerLane], const float (&b)[kAttnMaxDPerLane], int nd) {
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < kAttnMaxDPerLane; ++i)
    if (i < nd) s = fmaf(a[i], b[i], s);
  return wave_sum(s);
}

// The row statistics in the form the pipelined dK/dV walk copies straight into LDS: -lse in
// log2 units and -delta, each (B*H, s_pad) with s_pad a multiple of 64 and the rows past S
// holding -inf and 0 (probabilities of rows that do not exist vanish).  `idx` is the row's
// index in (B,H,S) order; the thread that owns a sequence's last row writes its padding.
struct AttnPaddedStats {
  const float* lse = nullptr;
  float* nlse = nullptr;    // null: not wanted
  float* ndelta = nullptr;
  int s_pad = 0;
};
__device__ __forceinline__ void write_padded_stats(const AttnPaddedStats& ps, int64_t idx, int S, float delta) {
  if (ps.nlse == nullptr) return;
  const int64_t bh = idx / S;
  const int s = static_cast<int>(idx - bh * S);
  ps.nlse[bh * ps.s_pad + s] = -ps.lse[idx] * kAttnLog2e;
  ps.ndelta[bh * ps.s_pad + s] = -delta;
  if (s == S - 1)
    for (int t = S; t < ps.s_pad; ++t) {
      ps.nlse[bh * ps.s_pad + t] = -INFINITY;
      ps.ndelta[bh * ps.s_pad + t] = 0.f;
    }
}

// delta[b,h,i] = sum_d dO[b,h,i,d] * O[b,h,i,d]
template <typename T>
__global__ __launch_bounds__(256) void attn_delta_kernel(const T* __restrict__ d_o, const T* __restrict__ o,
                                                         float* __restrict__ delta, int64_t rows, int D, int S, int H,
                                                         int o_bshd, AttnPaddedStats ps = {}) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (row >= rows) return;
  const int lane = threadIdx.x % kWave;
  float acc = 0.f;
  for (int d = lane; d < D; d += kWave) acc = fmaf(to_float(d_o[row * D + d]), to_float(o[row * D + d]), acc);
  acc = wave_sum(acc);
  if (lane == 0) {
    const int64_t idx = o_row_to_bhs(row, S, H, o_bshd);
    delta[idx] = acc;
    write_padded_stats(ps, idx, S, acc);
  }
}

// Forward: wave = one query row; online softmax in the exp2 domain.
template <typename T, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(256) void attn_fwd_generic_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                               const T* __restrict__ v, const T* __restrict__ mask,
                                                               T* __restrict__ o, float* __restrict__ lse, AttnDims a,
                                                               float scale) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;  // over B*H*S
  if (row >= static_cast<int64_t>(a.B) * a.H * a.S) return;
  const int lane = threadIdx.x % kWave;
  const int i = static_cast<int>(row % a.S);
  const int h = static_cast<int>((row / a.S) % a.H);
  const int b = static_cast<int>(row / (static_cast<int64_t>(a.S) * a.H));
  const int nd = (a.D + kWave - 1) / kWave;
  float qr[kAttnMaxDPerLane], acc[kAttnMaxDPerLane];
  load_row(q + qkv_at(a, b, i, h), a.D, lane, qr);
#pragma unroll
  for (int t = 0; t < kAttnMaxDPerLane; ++t) acc[t] = 0.f;
  const float c = scale * kAttnLog2e;
  float m = -INFINITY, l = 0.f;
  const int j_end = CAUSAL ? i + 1 : a.S;
  const T* mrow = HAS_BIAS ? mask + ((static_cast<int64_t>(b) * a.H + h) * a.S + i) * a.S : nullptr;
  for (int j = 0; j < j_end; ++j) {
    float kr[kAttnMaxDPerLane], vr[kAttnMaxDPerLane];
    load_row(k + qkv_at(a, b, j, h), a.D, lane, kr);
    load_row(v + qkv_at(a, b, j, h), a.D, lane, vr);
    float s = dot_rows(qr, kr, nd) * c;
    if (HAS_BIAS) s = fmaf(to_float(mrow[j]), kAttnLog2e, s);
    const float m_new = fmaxf(m, s);
    const float corr = exp2f(m - m_new);
    const float p = exp2f(s - m_new);
    l = l * corr + p;
#pragma unroll
    for (int t = 0; t < kAttnMaxDPerLane; ++t) acc[t] = fmaf(p, vr[t], acc[t] * corr);
    m = m_new;
  }
  const float inv = 1.0f / l;
  T* orow = o + o_at(a, b, h, i);
#pragma unroll
  for (int t = 0; t < kAttnMaxDPerLane; ++t) {
    const int d = lane + t * kWave;
    if (d < a.D) orow[d] = from_float<T>(acc[t] * inv);
  }
  if (lane == 0) lse[row] = m * kAttnLn2 + logf(l);
}

// dQ: wave = one query row.  P is recomputed from LSE.
template <typename T, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(256) void attn_dq_generic_kernel(const T* __restrict__ d_o, const T* __restrict__ q,
                                                              const T* __restrict__ k, const T* __restrict__ v,
                                                              const T* __restrict__ mask, const float* __restrict__ lse,
                                                              const float* __restrict__ delta, T* __restrict__ dq,
                                                              AttnDims a, float scale) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (row >= static_cast<int64_t>(a.B) * a.H * a.S) return;
  const int lane = threadIdx.x % kWave;
  const int i = static_cast<int>(row % a.S);
  const int h = static_cast<int>((row / a.S) % a.H);
  const int b = static_cast<int>(row / (static_cast<int64_t>(a.S) * a.H));
  const int nd = (a.D + kWave - 1) / kWave;
  float qr[kAttnMaxDPerLane], dor[kAttnMaxDPerLane], acc[kAttnMaxDPerLane];
  load_row(q + qkv_at(a, b, i, h), a.D, lane, qr);
  load_row(d_o + o_at(a, b, h, i), a.D, lane, dor);
#pragma unroll
  for (int t = 0; t < kAttnMaxDPerLane; ++t) acc[t] = 0.f;
  const float c = scale * kAttnLog2e;
  const float lse2 = lse[row] * kAttnLog2e;
  const float dl = delta[row];
  const int j_end = CAUSAL ? i + 1 : a.S;
  const T* mrow = HAS_BIAS ? mask + ((static_cast<int64_t>(b) * a.H + h) * a.S + i) * a.S : nullptr;
  for (int j = 0; j < j_end; ++j) {
    float kr[kAttnMaxDPerLane], vr[kAttnMaxDPerLane];
    load_row(k + qkv_at(a, b, j, h), a.D, lane, kr);
    load_row(v + qkv_at(a, b, j, h), a.D, lane, vr);
    float s = dot_rows(qr, kr, nd) * c;
    if (HAS_BIAS) s = fmaf(to_float(mrow[j]), kAttnLog2e, s);
    const float p = exp2f(s - lse2);
    const float dp = dot_rows(dor, vr, nd);
    const float ds = p * (dp - dl);
#pragma unroll
    for (int t = 0; t < kAttnMaxDPerLane; ++t) acc[t] = fmaf(ds, kr[t], acc[t]);
  }
  T* out = dq + qkv_at(a, b, i, h);
#pragma unroll
  for (int t = 0; t < kAttnMaxDPerLane; ++t) {
    const int d = lane + t * kWave;
    if (d < a.D) out[d] = from_float<T>(acc[t] * scale);
  }
}

// dK, dV: wave = one key row, loops over the query rows that see it.
template <typename T, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(256) void attn_dkdv_generic_kernel(const T* __restrict__ d_o, const T* __restrict__ q,
                                                                const T* __restrict__ k, const T* __restrict__ v,
                                                                const T* __restrict__ mask, const float* __restrict__ lse,
                                                                const float* __restrict__ delta, T* __restrict__ dk,
                                                                T* __restrict__ dv, AttnDims a, float scale) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (row >= static_cast<int64_t>(a.B) * a.H * a.S) return;
  const int lane = threadIdx.x % kWave;
  const int j = static_cast<int>(row % a.S);
  const int h = static_cast<int>((row / a.S) % a.H);
  const int b = static_cast<int>(row / (static_cast<int64_t>(a.S) * a.H));
  const int nd = (a.D + kWave - 1) / kWave;
  float kr[kAttnMaxDPerLane], vr[kAttnMaxDPerLane], acck[kAttnMaxDPerLane], accv[kAttnMaxDPerLane];
  load_row(k + qkv_at(a, b, j, h), a.D, lane, kr);
  load_row(v + qkv_at(a, b, j, h), a.D, lane, vr);
#pragma unroll
  for (int t = 0; t < kAttnMaxDPerLane; ++t) acck[t] = accv[t] = 0.f;
  const float c = scale * kAttnLog2e;
  const int64_t bh = static_cast<int64_t>(b) * a.H + h;
  const int i_begin = CAUSAL ? j : 0;
  for (int i = i_begin; i < a.S; ++i) {
    float qr[kAttnMaxDPerLane], dor[kAttnMaxDPerLane];
    load_row(q + qkv_at(a, b, i, h), a.D, lane, qr);
    load_row(d_o + o_at(a, b, h, i), a.D, lane, dor);
    float s = dot_rows(qr, kr, nd) * c;
    if (HAS_BIAS) s = fmaf(to_float(mask[(bh * a.S + i) * a.S + j]), kAttnLog2e, s);
    const float p = exp2f(s - lse[bh * a.S + i] * kAttnLog2e);
    const float dp = dot_rows(dor, vr, nd);
    const float ds = p * (dp - delta[bh * a.S + i]);
#pragma unroll
    for (int t = 0; t < kAttnMaxDPerLane; ++t) {
      accv[t] = fmaf(p, dor[t], accv[t]);
      acck[t] = fmaf(ds, qr[t], acck[t]);
    }
  }
  T* outk = dk + qkv_at(a, b, j, h);
  T* outv = dv + qkv_at(a, b, j, h);
#pragma unroll
  for (int t = 0; t < kAttnMaxDPerLane; ++t) {
    const int d = lane + t * kWave;
    if (d < a.D) {
      outk[d] = from_float<T>(acck[t] * scale);
      outv[d] = from_float<T>(accv[t]);
    }
  }
}

}  // namespace mg
