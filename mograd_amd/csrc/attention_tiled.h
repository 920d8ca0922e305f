// Flash attention in fp32 arithmetic for head dimensions up to 512, a row per thread (or per
// two to sixteen neighbouring threads): the form the general path takes when a sequence is
// long enough to fill workgroups.
//
// attention_generic.h gives every row a whole wave, one element of the head per lane, so each
// (query, key) pair costs a wave-wide reduction: about thirty instructions for 64 products.
// Here a thread keeps its row's slice of the head (DL elements, NT threads side by side share
// a row) in registers, a tile of TK rows of the other side's two tensors is staged in LDS as
// fp32 once per workgroup of 256 / NT rows, and every thread reads the same tile row at a
// time (an LDS broadcast).  A pair then costs two or three instructions per product and no
// cross-lane traffic beyond log2(NT) DPP additions, and K / V (or Q / dO) are fetched once
// per 256 / NT rows instead of once per row.  Same mathematics, masks, layouts and error
// budget as the wave-per-row kernels; fp32 FMA throughout, nothing of size S x S stored.
#pragma once

#include "attention_generic.h"

namespace mg {

// Sum over the NT neighbouring lanes that share a row (NT = 1 .. 16, a power of two: inside a
// quad, then across the quads of eight and of sixteen lanes by the mirrored moves).
template <int NT>
__device__ __forceinline__ float row_lanes_sum(float v) {
  static_assert(NT == 1 || NT == 2 || NT == 4 || NT == 8 || NT == 16, "lanes per row");
  if constexpr (NT >= 2) v += dpp_move<kDppQuadXor1>(v);
  if constexpr (NT >= 4) v += dpp_move<kDppQuadXor2>(v);
  if constexpr (NT >= 8) v += dpp_move<kDppRowHalfMirror>(v);
  if constexpr (NT >= 16) v += dpp_move<kDppRowMirror>(v);
  return v;
}

// Rows of a staged tile: 2048 / (NT * DL) of them, so that a tile is 8 KB per tensor, and at
// least the eight keys that the forward handles at a time.
template <int NT, int DL>
constexpr int tiled_rows() { return 2048 / (NT * DL) < 8 ? 8 : 2048 / (NT * DL); }

// Stage TK rows (first row j0, row stride `ld` elements, rows >= S and columns >= D as zeros)
// of `src` into `dst` [TK][NT * DL] as fp32, all 256 threads taking part.
template <typename T, int NT, int DL>
__device__ __forceinline__ void tiled_stage(const T* __restrict__ src, int64_t ld, int j0, int S, int D,
                                            float* __restrict__ dst) {
  constexpr int DP = NT * DL, TK = tiled_rows<NT, DL>();
  for (int e = threadIdx.x; e < TK * DP; e += 256) {
    const int jj = e / DP, d = e % DP;
    const int j = j0 + jj;
    dst[e] = (j < S && d < D) ? to_float(src[static_cast<int64_t>(j) * ld + d]) : 0.f;
  }
}

// This thread's DL-element slice of a row, as fp32, times `f`; zeros past D or past the end.
template <typename T, int DL>
__device__ __forceinline__ void tiled_load_slice(const T* __restrict__ row, bool row_ok, int d0, int D, float f,
                                                 float (&v)[DL]) {
#pragma unroll
  for (int d = 0; d < DL; ++d) v[d] = (row_ok && d0 + d < D) ? to_float(row[d0 + d]) * f : 0.f;
}

template <int DL>
__device__ __forceinline__ float tiled_dot(const float (&a)[DL], const float* __restrict__ b) {
  float s = 0.f;
#pragma unroll
  for (int d = 0; d < DL; d += 4) {
    const float4 w = *reinterpret_cast<const float4*>(b + d);
    s = fmaf(a[d], w.x, s);
    s = fmaf(a[d + 1], w.y, s);
    s = fmaf(a[d + 2], w.z, s);
    s = fmaf(a[d + 3], w.w, s);
  }
  return s;
}
template <int DL>
__device__ __forceinline__ void tiled_axpy(float f, const float* __restrict__ b, float (&acc)[DL]) {
#pragma unroll
  for (int d = 0; d < DL; d += 4) {
    const float4 w = *reinterpret_cast<const float4*>(b + d);
    acc[d] = fmaf(f, w.x, acc[d]);
    acc[d + 1] = fmaf(f, w.y, acc[d + 1]);
    acc[d + 2] = fmaf(f, w.z, acc[d + 2]);
    acc[d + 3] = fmaf(f, w.w, acc[d + 3]);
  }
}

// Forward.  Grid (query blocks of 256 / NT rows, B * H).  Online softmax per thread, one
// rescale of the accumulators per eight keys.
template <typename T, int NT, int DL, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(256, 2) void attn_fwd_tiled_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                             const T* __restrict__ v, const T* __restrict__ mask,
                                                             T* __restrict__ o, float* __restrict__ lse, AttnDims a,
                                                             float scale) {
  constexpr int DP = NT * DL, TK = tiled_rows<NT, DL>(), R = 256 / NT;
  __shared__ __attribute__((aligned(16))) float k_s[TK * DP];
  __shared__ __attribute__((aligned(16))) float v_s[TK * DP];
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const int r0 = blockIdx.x * R;
  const int i = r0 + threadIdx.x / NT, d0 = (threadIdx.x % NT) * DL;
  const bool row_ok = i < a.S;
  float qr[DL], acc[DL];
  tiled_load_slice<T, DL>(q + qkv_at(a, b, min(i, a.S - 1), h), row_ok, d0, a.D, scale * kAttnLog2e, qr);
#pragma unroll
  for (int d = 0; d < DL; ++d) acc[d] = 0.f;
  float m = -INFINITY, l = 0.f;
  const int j_end = CAUSAL ? min(a.S, r0 + R) : a.S;
  const T* kbase = k + qkv_at(a, b, 0, h);
  const T* vbase = v + qkv_at(a, b, 0, h);
  const T* mrow = HAS_BIAS ? mask + (static_cast<int64_t>(bh) * a.S + min(i, a.S - 1)) * a.S : nullptr;
  for (int j0 = 0; j0 < j_end; j0 += TK) {
    __syncthreads();  // every thread is done with the previous tile
    tiled_stage<T, NT, DL>(kbase, a.ld, j0, a.S, a.D, k_s);
    tiled_stage<T, NT, DL>(vbase, a.ld, j0, a.S, a.D, v_s);
    __syncthreads();
    // eight keys at a time: their scores, one rescale of the accumulators, their values
#pragma unroll 1
    for (int j8 = 0; j8 < TK; j8 += 8) {
      float s[8];
      float m_new = m;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int jj = j8 + u, j = j0 + jj;
        float sv = row_lanes_sum<NT>(tiled_dot<DL>(qr, k_s + jj * DP + d0));
        if (HAS_BIAS) sv = fmaf(to_float(mrow[min(j, a.S - 1)]), kAttnLog2e, sv);
        const bool valid = j < a.S && (!CAUSAL || j <= i);
        s[u] = valid ? sv : -INFINITY;
        m_new = fmaxf(m_new, s[u]);
      }
      if (m_new == -INFINITY) continue;  // nothing visible yet
      const float corr = exp2f(m - m_new);
      l *= corr;
#pragma unroll
      for (int d = 0; d < DL; ++d) acc[d] *= corr;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float p = exp2f(s[u] - m_new);
        l += p;
        tiled_axpy<DL>(p, v_s + (j8 + u) * DP + d0, acc);
      }
      m = m_new;
    }
  }
  if (!row_ok) return;
  const float inv = 1.0f / l;
  T* orow = o + o_at(a, b, h, i);
#pragma unroll
  for (int d = 0; d < DL; ++d)
    if (d0 + d < a.D) orow[d0 + d] = from_float<T>(acc[d] * inv);
  if (threadIdx.x % NT == 0) lse[static_cast<int64_t>(bh) * a.S + i] = m * kAttnLn2 + logf(l);
}

// dQ.  Grid as the forward; P is recomputed from LSE.
template <typename T, int NT, int DL, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(256, 2) void attn_dq_tiled_kernel(const T* __restrict__ d_o, const T* __restrict__ q,
                                                            const T* __restrict__ k, const T* __restrict__ v,
                                                            const T* __restrict__ mask, const float* __restrict__ lse,
                                                            const float* __restrict__ delta, T* __restrict__ dq,
                                                            AttnDims a, float scale) {
  constexpr int DP = NT * DL, TK = tiled_rows<NT, DL>(), R = 256 / NT;
  __shared__ __attribute__((aligned(16))) float k_s[TK * DP];
  __shared__ __attribute__((aligned(16))) float v_s[TK * DP];
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const int r0 = blockIdx.x * R;
  const int i = r0 + threadIdx.x / NT, d0 = (threadIdx.x % NT) * DL;
  const bool row_ok = i < a.S;
  const int ic = min(i, a.S - 1);
  float qr[DL], dor[DL], acc[DL];
  tiled_load_slice<T, DL>(q + qkv_at(a, b, ic, h), row_ok, d0, a.D, scale * kAttnLog2e, qr);
  tiled_load_slice<T, DL>(d_o + o_at(a, b, h, ic), row_ok, d0, a.D, 1.0f, dor);
#pragma unroll
  for (int d = 0; d < DL; ++d) acc[d] = 0.f;
  const float lse2 = row_ok ? lse[static_cast<int64_t>(bh) * a.S + i] * kAttnLog2e : INFINITY;
  const float dl = row_ok ? delta[static_cast<int64_t>(bh) * a.S + i] : 0.f;
  const int j_end = CAUSAL ? min(a.S, r0 + R) : a.S;
  const T* kbase = k + qkv_at(a, b, 0, h);
  const T* vbase = v + qkv_at(a, b, 0, h);
  const T* mrow = HAS_BIAS ? mask + (static_cast<int64_t>(bh) * a.S + ic) * a.S : nullptr;
  for (int j0 = 0; j0 < j_end; j0 += TK) {
    __syncthreads();
    tiled_stage<T, NT, DL>(kbase, a.ld, j0, a.S, a.D, k_s);
    tiled_stage<T, NT, DL>(vbase, a.ld, j0, a.S, a.D, v_s);
    __syncthreads();
#pragma unroll 1
    for (int jj = 0; jj < TK; ++jj) {
      const int j = j0 + jj;
      float sv = row_lanes_sum<NT>(tiled_dot<DL>(qr, k_s + jj * DP + d0));
      if (HAS_BIAS) sv = fmaf(to_float(mrow[min(j, a.S - 1)]), kAttnLog2e, sv);
      const bool valid = j < a.S && (!CAUSAL || j <= i);
      const float p = valid ? exp2f(sv - lse2) : 0.f;
      const float dp = row_lanes_sum<NT>(tiled_dot<DL>(dor, v_s + jj * DP + d0));
      // K was staged unscaled and Q scaled by scale * log2(e): dS K scale is formed at the end
      tiled_axpy<DL>(p * (dp - dl), k_s + jj * DP + d0, acc);
    }
  }
  if (!row_ok) return;
  T* out = dq + qkv_at(a, b, i, h);
#pragma unroll
  for (int d = 0; d < DL; ++d)
    if (d0 + d < a.D) out[d0 + d] = from_float<T>(acc[d] * scale);
}

// dK, dV.  Grid (key blocks of 256 / NT rows, B * H); the query rows that see the block are
// streamed with their statistics.
template <typename T, int NT, int DL, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(256, 2) void attn_dkdv_tiled_kernel(const T* __restrict__ d_o, const T* __restrict__ q,
                                                              const T* __restrict__ k, const T* __restrict__ v,
                                                              const T* __restrict__ mask, const float* __restrict__ lse,
                                                              const float* __restrict__ delta, T* __restrict__ dk,
                                                              T* __restrict__ dv, AttnDims a, float scale) {
  constexpr int DP = NT * DL, TK = tiled_rows<NT, DL>(), R = 256 / NT;
  __shared__ __attribute__((aligned(16))) float q_s[TK * DP];
  __shared__ __attribute__((aligned(16))) float do_s[TK * DP];
  __shared__ float lse_s[TK], delta_s[TK];
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const int r0 = blockIdx.x * R;
  const int j = r0 + threadIdx.x / NT, d0 = (threadIdx.x % NT) * DL;
  const bool row_ok = j < a.S;
  const int jc = min(j, a.S - 1);
  float kr[DL], vr[DL], acck[DL], accv[DL];
  tiled_load_slice<T, DL>(k + qkv_at(a, b, jc, h), row_ok, d0, a.D, scale * kAttnLog2e, kr);
  tiled_load_slice<T, DL>(v + qkv_at(a, b, jc, h), row_ok, d0, a.D, 1.0f, vr);
#pragma unroll
  for (int d = 0; d < DL; ++d) acck[d] = accv[d] = 0.f;
  const T* qbase = q + qkv_at(a, b, 0, h);
  const T* dobase = d_o + o_at(a, b, h, 0);
  const int i_begin = CAUSAL ? (r0 / TK) * TK : 0;
  for (int i0 = i_begin; i0 < a.S; i0 += TK) {
    __syncthreads();
    tiled_stage<T, NT, DL>(qbase, a.ld, i0, a.S, a.D, q_s);
    tiled_stage<T, NT, DL>(dobase, o_ld(a), i0, a.S, a.D, do_s);
    if (threadIdx.x < TK) {
      const int i = i0 + threadIdx.x;
      // rows past the end get lse = +inf: their probabilities vanish
      lse_s[threadIdx.x] = i < a.S ? lse[static_cast<int64_t>(bh) * a.S + i] * kAttnLog2e : INFINITY;
      delta_s[threadIdx.x] = i < a.S ? delta[static_cast<int64_t>(bh) * a.S + i] : 0.f;
    }
    __syncthreads();
#pragma unroll 1
    for (int ii = 0; ii < TK; ++ii) {
      const int i = i0 + ii;
      float sv = row_lanes_sum<NT>(tiled_dot<DL>(kr, q_s + ii * DP + d0));
      if (HAS_BIAS) sv = fmaf(to_float(mask[(static_cast<int64_t>(bh) * a.S + min(i, a.S - 1)) * a.S + jc]), kAttnLog2e, sv);
      const bool valid = i < a.S && (!CAUSAL || j <= i);
      const float p = valid ? exp2f(sv - lse_s[ii]) : 0.f;
      const float dp = row_lanes_sum<NT>(tiled_dot<DL>(vr, do_s + ii * DP + d0));
      tiled_axpy<DL>(p, do_s + ii * DP + d0, accv);
      tiled_axpy<DL>(p * (dp - delta_s[ii]), q_s + ii * DP + d0, acck);
    }
  }
  if (!row_ok) return;
  T* outk = dk + qkv_at(a, b, j, h);
  T* outv = dv + qkv_at(a, b, j, h);
#pragma unroll
  for (int d = 0; d < DL; ++d)
    if (d0 + d < a.D) {
      outk[d0 + d] = from_float<T>(acck[d] * scale);
      outv[d0 + d] = from_float<T>(accv[d]);
    }
}

}  // namespace mg
