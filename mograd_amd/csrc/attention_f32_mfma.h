// Flash attention in fp32 arithmetic on the matrix cores (v_mfma_f32_32x32x2_f32), head
// dimensions up to 128 (kernels for 32, 64 and 128 columns): what fp32 tensors take once a
// sequence fills a workgroup.
//
// The row-per-thread kernels of attention_tiled.h reach a third of the fp32 FMA rate; the fp32
// MFMA has twice that rate and leaves the VALU to the softmax.  Layout of a 32 x 32 x 2 product:
// lane l supplies A[row = l % 32][k = l / 32] and B[k = l / 32][col = l % 32] and receives
// column l % 32 of the result, sixteen rows (r/4)*8 + (l/32)*4 + r%4.  Three consequences carry
// the kernels:
//  - which two elements of the contraction a step multiplies is free as long as A and B agree,
//    so step s takes head columns s (lower half wave) and DP/2 + s (upper half): a lane's DP/2
//    values of a resident row, and of a streamed row, are contiguous in memory;
//  - a score tile computed with the resident rows along the lanes comes out as "lane = resident
//    row, registers = streamed rows", which is the B operand of the products that contract
//    over the streamed rows (O = P V, dQ = dS K, dV = P^T dO, dK = dS^T Q): register j of a lane
//    is its k-slice of step j, so P and dS never leave registers;
//  - the softmax statistics of a resident row are per lane (forward, dQ), those of a streamed row
//    per register (dK/dV).
// A workgroup is four waves of 32 resident rows each; tiles of 32 streamed rows of two tensors go
// through LDS as fp32 (rows padded by four floats: the 128-bit reads of sixteen rows then fall in
// sixteen different bank groups), fetched into registers one tile ahead (a second copy of the tiles
// in LDS, which saves one of the two barriers per step, measured no faster: the steps are bound by the
// matrix pipe, not by the barriers).  The 128-column kernels
// run one workgroup per CU with the 512-register budget (two resident rows of 64 values and
// eight accumulators per lane in dK/dV).  Same mathematics, masks,
// layouts, LSE and error budget as the other fp32 forms; nothing of size S x S is stored.
#pragma once

#include "attention_generic.h"

namespace mg {

constexpr int kF32AttnMaxD = 128;   // widest head these kernels take
constexpr int kF32AttnRows = 32;    // streamed rows per step
constexpr int kF32AttnBlock = 128;  // resident rows per workgroup

typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ f32x16 f32_mfma(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 f32x16_zero() {
  f32x16 z;
#pragma unroll
  for (int r = 0; r < 16; ++r) z[r] = 0.f;
  return z;
}
// Row, inside a 32-row tile, of accumulator register r of a lane in half `half`.
__device__ __forceinline__ int f32_acc_row(int r, int half) { return (r / 4) * 8 + half * 4 + r % 4; }

// Four consecutive elements of a row as fp32 (zeros for a missing row or columns past D).
template <typename T>
__device__ __forceinline__ float4 f32_attn_load4(const T* __restrict__ row, bool row_ok, int d, int D, bool vec_ok) {
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (!row_ok) return v;
  if constexpr (sizeof(T) == 4) {
    if (vec_ok && d + 4 <= D) return *reinterpret_cast<const float4*>(row + d);
  }
  if (d < D) v.x = to_float(row[d]);
  if (d + 1 < D) v.y = to_float(row[d + 1]);
  if (d + 2 < D) v.z = to_float(row[d + 2]);
  if (d + 3 < D) v.w = to_float(row[d + 3]);
  return v;
}

// A lane's DP / 2 values of a resident row: columns half * DP / 2 onwards, times f.
template <typename T, int DP>
__device__ __forceinline__ void f32_attn_resident(const T* __restrict__ row, bool row_ok, int half, int D, float f,
                                                  bool vec_ok, float (&v)[DP / 2]) {
#pragma unroll
  for (int c = 0; c < DP / 8; ++c) {
    const float4 w = f32_attn_load4<T>(row, row_ok, half * (DP / 2) + c * 4, D, vec_ok);
    v[c * 4] = w.x * f;
    v[c * 4 + 1] = w.y * f;
    v[c * 4 + 2] = w.z * f;
    v[c * 4 + 3] = w.w * f;
  }
}

// The streamed tile pair of a step in flight: thread t holds chunks t, t + 256, ... (a chunk is
// four columns; DP / 4 consecutive threads cover a row) of both tensors.
template <int DP>
struct F32AttnStage {
  float4 a[DP / 32], b[DP / 32];
};
template <typename T, int DP>
__device__ __forceinline__ void f32_attn_fetch(const T* __restrict__ ta, int64_t lda, const T* __restrict__ tb, int64_t ldb,
                                               int row0, int S, int D, bool vec_ok, F32AttnStage<DP>& st) {
#pragma unroll
  for (int u = 0; u < DP / 32; ++u) {
    const int e = threadIdx.x + 256 * u, rr = e / (DP / 4), ch = e % (DP / 4);
    const int row = row0 + rr;
    const bool ok = row < S;
    st.a[u] = f32_attn_load4<T>(ta + static_cast<int64_t>(row) * lda, ok, ch * 4, D, vec_ok);
    st.b[u] = f32_attn_load4<T>(tb + static_cast<int64_t>(row) * ldb, ok, ch * 4, D, vec_ok);
  }
}
template <int DP>
__device__ __forceinline__ void f32_attn_commit(const F32AttnStage<DP>& st, float* __restrict__ a_s,
                                                float* __restrict__ b_s) {
#pragma unroll
  for (int u = 0; u < DP / 32; ++u) {
    const int e = threadIdx.x + 256 * u, rr = e / (DP / 4), ch = e % (DP / 4);
    *reinterpret_cast<float4*>(a_s + rr * (DP + 4) + ch * 4) = st.a[u];
    *reinterpret_cast<float4*>(b_s + rr * (DP + 4) + ch * 4) = st.b[u];
  }
}

// acc += tile * resident^T: rows of the tile along the result's rows, the wave's resident rows
// along its columns (lanes); the contraction runs over the DP head columns.
template <int DP>
__device__ __forceinline__ f32x16 f32_attn_scores(const float* __restrict__ tile, const float (&resident)[DP / 2], int lane,
                                                  f32x16 acc) {
  const float* mine = tile + (lane % 32) * (DP + 4) + (lane / 32) * (DP / 2);
#pragma unroll
  for (int c = 0; c < DP / 8; ++c) {
    const float4 w = *reinterpret_cast<const float4*>(mine + c * 4);
    acc = f32_mfma(w.x, resident[c * 4], acc);
    acc = f32_mfma(w.y, resident[c * 4 + 1], acc);
    acc = f32_mfma(w.z, resident[c * 4 + 2], acc);
    acc = f32_mfma(w.w, resident[c * 4 + 3], acc);
  }
  return acc;
}

// out[db] += tile^T (columns db * 32 .. + 31 along the result's rows) * w, where w is a score
// tile in accumulator layout (register j = the lane's k-slice of step j); the contraction runs
// over the tile's 32 rows.
template <int DP>
__device__ __forceinline__ void f32_attn_weighted(const float* __restrict__ tile, const f32x16& w, int lane,
                                                  f32x16 (&out)[DP / 32]) {
  const int half = lane / 32;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const float* row = tile + f32_acc_row(j, half) * (DP + 4) + lane % 32;
#pragma unroll
    for (int db = 0; db < DP / 32; ++db) out[db] = f32_mfma(row[db * 32], w[j], out[db]);
  }
}

// The lane's resident row gets columns db * 32 + f32_acc_row(r, half) of its result: groups of
// four consecutive columns per four registers.
template <typename T, int DP>
__device__ __forceinline__ void f32_attn_store(T* __restrict__ row, const f32x16 (&acc)[DP / 32], float f, int half, int D,
                                               bool vec_ok) {
#pragma unroll
  for (int db = 0; db < DP / 32; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = db * 32 + g * 8 + half * 4;
      const float v0 = acc[db][g * 4] * f, v1 = acc[db][g * 4 + 1] * f, v2 = acc[db][g * 4 + 2] * f,
                  v3 = acc[db][g * 4 + 3] * f;
      if constexpr (sizeof(T) == 4) {
        if (vec_ok && d + 4 <= D) {
          *reinterpret_cast<float4*>(row + d) = make_float4(v0, v1, v2, v3);
          continue;
        }
      }
      if (d < D) row[d] = from_float<T>(v0);
      if (d + 1 < D) row[d + 1] = from_float<T>(v1);
      if (d + 2 < D) row[d + 2] = from_float<T>(v2);
      if (d + 3 < D) row[d + 3] = from_float<T>(v3);
    }
}

// Bias of (row i, columns j0 + f32_acc_row(r, half)) for the sixteen registers, as loaded: any
// arithmetic on the values here would put the wait for them in front of the products that are
// meant to hide it.
template <typename T>
__device__ __forceinline__ void f32_attn_bias_row(const T* __restrict__ mrow, int j0, int half, int S, bool vec_ok,
                                                  float (&b)[16]) {
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int j = j0 + g * 8 + half * 4;
    if constexpr (sizeof(T) == 4) {
      if (vec_ok && j + 4 <= S) {
        const float4 w = *reinterpret_cast<const float4*>(mrow + j);
        b[g * 4] = w.x;
        b[g * 4 + 1] = w.y;
        b[g * 4 + 2] = w.z;
        b[g * 4 + 3] = w.w;
        continue;
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) b[g * 4 + e] = to_float(mrow[min(j + e, S - 1)]);
  }
}

__device__ __forceinline__ bool f32_attn_vec_ok(const void* p, int64_t ld, int D) {
  return D % 4 == 0 && ld % 4 == 0 && reinterpret_cast<uintptr_t>(p) % 16 == 0;
}

// Forward.  Grid (B * H, query blocks of 128): the heads of one block position run side by side, and a
// causal launch starts with the last positions, whose walks are the longest.  Scores come out as
// keys x queries, so a query's
// maximum and sum are over a lane's sixteen registers and its partner lane in the other half.
template <typename T, int DP, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(256, DP > 64 ? 1 : 2) void attn_fwd_f32_mfma_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, const T* __restrict__ mask,
    T* __restrict__ o, float* __restrict__ lse, AttnDims a, float scale) {
  __shared__ __attribute__((aligned(16))) float k_s[kF32AttnRows * (DP + 4)];
  __shared__ __attribute__((aligned(16))) float v_s[kF32AttnRows * (DP + 4)];
  const int bh = blockIdx.x, b = bh / a.H, h = bh % a.H;
  const int r0 = (CAUSAL ? gridDim.y - 1 - blockIdx.y : blockIdx.y) * kF32AttnBlock;  // longest walks first
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave, half = lane / 32;
  const int i = r0 + wave * 32 + lane % 32;
  const bool row_ok = i < a.S;
  const int ic = min(i, a.S - 1);
  const bool vec_qkv = f32_attn_vec_ok(q, a.ld, a.D) && f32_attn_vec_ok(k, a.ld, a.D) && f32_attn_vec_ok(v, a.ld, a.D);
  const bool vec_o = f32_attn_vec_ok(o, o_ld(a), a.D);
  const bool vec_m = HAS_BIAS && a.S % 4 == 0 && reinterpret_cast<uintptr_t>(mask) % 16 == 0;
  float qr[DP / 2];
  f32_attn_resident<T, DP>(q + qkv_at(a, b, ic, h), row_ok, half, a.D, scale * kAttnLog2e, vec_qkv, qr);
  f32x16 acc[DP / 32];
#pragma unroll
  for (int db = 0; db < DP / 32; ++db) acc[db] = f32x16_zero();
  float m = -INFINITY, l = 0.f;  // l: this lane's half of the row's sum
  const int j_end = CAUSAL ? min(a.S, r0 + kF32AttnBlock) : a.S;
  const int wave_last = r0 + wave * 32 + 31;  // last query of the wave
  const T* kbase = k + qkv_at(a, b, 0, h);
  const T* vbase = v + qkv_at(a, b, 0, h);
  const T* mrow = HAS_BIAS ? mask + (static_cast<int64_t>(bh) * a.S + ic) * a.S : nullptr;
  F32AttnStage<DP> st;
  f32_attn_fetch<T, DP>(kbase, a.ld, vbase, a.ld, 0, a.S, a.D, vec_qkv, st);
  for (int j0 = 0; j0 < j_end; j0 += kF32AttnRows) {
    __syncthreads();  // every wave is done with the previous tile
    f32_attn_commit<DP>(st, k_s, v_s);
    __syncthreads();
    if (j0 + kF32AttnRows < j_end) f32_attn_fetch<T, DP>(kbase, a.ld, vbase, a.ld, j0 + kF32AttnRows, a.S, a.D, vec_qkv, st);
    if (CAUSAL && j0 > wave_last) continue;  // wave-uniform: nothing of this tile is visible
    float bias[16];  // requested before the products that hide the loads (and kept there)
    if (HAS_BIAS) {
      f32_attn_bias_row<T>(mrow, j0, half, a.S, vec_m, bias);
      __builtin_amdgcn_sched_barrier(0);
    }
    f32x16 s = f32_attn_scores<DP>(k_s, qr, lane, f32x16_zero());
    float m_tile = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = j0 + f32_acc_row(r, half);
      float sv = s[r];
      if (HAS_BIAS) sv = fmaf(bias[r], kAttnLog2e, sv);
      const bool valid = j < a.S && (!CAUSAL || j <= i);
      s[r] = valid ? sv : -INFINITY;
      m_tile = fmaxf(m_tile, s[r]);
    }
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32));
    const float m_new = fmaxf(m, m_tile);
    if (m_new == -INFINITY) {  // nothing visible to this row yet: its weights are zero
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.f;
    } else {
      const float corr = exp2f(m - m_new);
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        s[r] = exp2f(s[r] - m_new);
        sum += s[r];
      }
      l = l * corr + sum;
#pragma unroll
      for (int db = 0; db < DP / 32; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[db][r] *= corr;
      m = m_new;
    }
    f32_attn_weighted<DP>(v_s, s, lane, acc);
  }
  const float l_row = l + __shfl_xor(l, 32);
  if (!row_ok) return;
  f32_attn_store<T, DP>(o + o_at(a, b, h, i), acc, 1.0f / l_row, half, a.D, vec_o);
  if (half == 0) lse[static_cast<int64_t>(bh) * a.S + i] = m * kAttnLn2 + logf(l_row);
}

// dQ.  Grid as the forward; P is recomputed from LSE, dP = V dO^T comes out in the same layout.
template <typename T, int DP, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(256, DP > 64 ? 1 : 2) void attn_dq_f32_mfma_kernel(
    const T* __restrict__ d_o, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const T* __restrict__ mask, const float* __restrict__ lse, const float* __restrict__ delta, T* __restrict__ dq,
    AttnDims a, float scale) {
  __shared__ __attribute__((aligned(16))) float k_s[kF32AttnRows * (DP + 4)];
  __shared__ __attribute__((aligned(16))) float v_s[kF32AttnRows * (DP + 4)];
  const int bh = blockIdx.x, b = bh / a.H, h = bh % a.H;
  const int r0 = (CAUSAL ? gridDim.y - 1 - blockIdx.y : blockIdx.y) * kF32AttnBlock;  // longest walks first
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave, half = lane / 32;
  const int i = r0 + wave * 32 + lane % 32;
  const bool row_ok = i < a.S;
  const int ic = min(i, a.S - 1);
  const bool vec_qkv = f32_attn_vec_ok(q, a.ld, a.D) && f32_attn_vec_ok(k, a.ld, a.D) && f32_attn_vec_ok(v, a.ld, a.D) &&
                       f32_attn_vec_ok(dq, a.ld, a.D);
  const bool vec_o = f32_attn_vec_ok(d_o, o_ld(a), a.D);
  const bool vec_m = HAS_BIAS && a.S % 4 == 0 && reinterpret_cast<uintptr_t>(mask) % 16 == 0;
  float qr[DP / 2], dor[DP / 2];
  f32_attn_resident<T, DP>(q + qkv_at(a, b, ic, h), row_ok, half, a.D, scale * kAttnLog2e, vec_qkv, qr);
  f32_attn_resident<T, DP>(d_o + o_at(a, b, h, ic), row_ok, half, a.D, 1.0f, vec_o, dor);
  f32x16 acc[DP / 32];
#pragma unroll
  for (int db = 0; db < DP / 32; ++db) acc[db] = f32x16_zero();
  const float lse2 = row_ok ? lse[static_cast<int64_t>(bh) * a.S + i] * kAttnLog2e : INFINITY;
  const float dl = row_ok ? delta[static_cast<int64_t>(bh) * a.S + i] : 0.f;
  const int j_end = CAUSAL ? min(a.S, r0 + kF32AttnBlock) : a.S;
  const int wave_last = r0 + wave * 32 + 31;
  const T* kbase = k + qkv_at(a, b, 0, h);
  const T* vbase = v + qkv_at(a, b, 0, h);
  const T* mrow = HAS_BIAS ? mask + (static_cast<int64_t>(bh) * a.S + ic) * a.S : nullptr;
  F32AttnStage<DP> st;
  f32_attn_fetch<T, DP>(kbase, a.ld, vbase, a.ld, 0, a.S, a.D, vec_qkv, st);
  for (int j0 = 0; j0 < j_end; j0 += kF32AttnRows) {
    __syncthreads();
    f32_attn_commit<DP>(st, k_s, v_s);
    __syncthreads();
    if (j0 + kF32AttnRows < j_end) f32_attn_fetch<T, DP>(kbase, a.ld, vbase, a.ld, j0 + kF32AttnRows, a.S, a.D, vec_qkv, st);
    if (CAUSAL && j0 > wave_last) continue;
    float bias[16];
    if (HAS_BIAS) {
      f32_attn_bias_row<T>(mrow, j0, half, a.S, vec_m, bias);
      __builtin_amdgcn_sched_barrier(0);
    }
    f32x16 s = f32_attn_scores<DP>(k_s, qr, lane, f32x16_zero());
    const f32x16 dp = f32_attn_scores<DP>(v_s, dor, lane, f32x16_zero());
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = j0 + f32_acc_row(r, half);
      float sv = s[r];
      if (HAS_BIAS) sv = fmaf(bias[r], kAttnLog2e, sv);
      const bool valid = j < a.S && (!CAUSAL || j <= i);
      const float p = valid ? exp2f(sv - lse2) : 0.f;
      s[r] = p * (dp[r] - dl);  // dS without the scale: K was staged unscaled, the scale goes on at the end
    }
    f32_attn_weighted<DP>(k_s, s, lane, acc);
  }
  if (!row_ok) return;
  f32_attn_store<T, DP>(dq + qkv_at(a, b, i, h), acc, scale, half, a.D, vec_qkv);
}

// dK, dV.  Grid (B * H, key blocks of 128).  The wave's keys are along the lanes, the streamed
// queries along the registers, so LSE and delta of a tile's rows are read per register.
template <typename T, int DP, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(256, DP > 64 ? 1 : 2) void attn_dkdv_f32_mfma_kernel(
    const T* __restrict__ d_o, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const T* __restrict__ mask, const float* __restrict__ lse, const float* __restrict__ delta, T* __restrict__ dk,
    T* __restrict__ dv, AttnDims a, float scale) {
  __shared__ __attribute__((aligned(16))) float q_s[kF32AttnRows * (DP + 4)];
  __shared__ __attribute__((aligned(16))) float do_s[kF32AttnRows * (DP + 4)];
  __shared__ __attribute__((aligned(16))) float lse_s[kF32AttnRows];
  __shared__ __attribute__((aligned(16))) float delta_s[kF32AttnRows];
  const int bh = blockIdx.x, b = bh / a.H, h = bh % a.H;
  const int r0 = blockIdx.y * kF32AttnBlock;  // causal: the first key blocks have the longest walks
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave, half = lane / 32;
  const int j = r0 + wave * 32 + lane % 32;
  const bool row_ok = j < a.S;
  const int jc = min(j, a.S - 1);
  const bool vec_qkv = f32_attn_vec_ok(q, a.ld, a.D) && f32_attn_vec_ok(k, a.ld, a.D) && f32_attn_vec_ok(v, a.ld, a.D) &&
                       f32_attn_vec_ok(dk, a.ld, a.D) && f32_attn_vec_ok(dv, a.ld, a.D);
  const bool vec_o = f32_attn_vec_ok(d_o, o_ld(a), a.D);
  float kr[DP / 2], vr[DP / 2];
  f32_attn_resident<T, DP>(k + qkv_at(a, b, jc, h), row_ok, half, a.D, scale * kAttnLog2e, vec_qkv, kr);
  f32_attn_resident<T, DP>(v + qkv_at(a, b, jc, h), row_ok, half, a.D, 1.0f, vec_qkv, vr);
  f32x16 acck[DP / 32], accv[DP / 32];
#pragma unroll
  for (int db = 0; db < DP / 32; ++db) acck[db] = accv[db] = f32x16_zero();
  const T* qbase = q + qkv_at(a, b, 0, h);
  const T* dobase = d_o + o_at(a, b, h, 0);
  const int64_t ldo = o_ld(a);
  const bool vec_both = vec_qkv && vec_o;
  const int i_begin = CAUSAL ? (r0 / kF32AttnRows) * kF32AttnRows : 0;
  const int wave_first = r0 + wave * 32;  // first key of the wave
  F32AttnStage<DP> st;
  float st_lse = 0.f, st_delta = 0.f;
  auto fetch = [&](int i0) {
    f32_attn_fetch<T, DP>(qbase, a.ld, dobase, ldo, i0, a.S, a.D, vec_both, st);
    if (threadIdx.x < kF32AttnRows) {
      const int i = i0 + threadIdx.x;
      // rows past the end get lse = +inf: their probabilities vanish
      st_lse = i < a.S ? lse[static_cast<int64_t>(bh) * a.S + i] * kAttnLog2e : INFINITY;
      st_delta = i < a.S ? delta[static_cast<int64_t>(bh) * a.S + i] : 0.f;
    }
  };
  fetch(i_begin);
  for (int i0 = i_begin; i0 < a.S; i0 += kF32AttnRows) {
    __syncthreads();
    f32_attn_commit<DP>(st, q_s, do_s);
    if (threadIdx.x < kF32AttnRows) {
      lse_s[threadIdx.x] = st_lse;
      delta_s[threadIdx.x] = st_delta;
    }
    __syncthreads();
    if (i0 + kF32AttnRows < a.S) fetch(i0 + kF32AttnRows);
    if (CAUSAL && i0 + kF32AttnRows - 1 < wave_first) continue;  // wave-uniform: no query of the tile sees these keys
    float bias[16];  // rows i0 + f32_acc_row(r, half) of the bias, this lane's key column
    if (HAS_BIAS) {
      const T* mcol = mask + static_cast<int64_t>(bh) * a.S * a.S + jc;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        bias[r] = to_float(mcol[static_cast<int64_t>(min(i0 + f32_acc_row(r, half), a.S - 1)) * a.S]);
      __builtin_amdgcn_sched_barrier(0);
    }
    f32x16 s = f32_attn_scores<DP>(q_s, kr, lane, f32x16_zero());
    f32x16 dp = f32_attn_scores<DP>(do_s, vr, lane, f32x16_zero());
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int rr = g * 8 + half * 4;
      const float4 l4 = *reinterpret_cast<const float4*>(lse_s + rr);
      const float4 d4 = *reinterpret_cast<const float4*>(delta_s + rr);
      const float lv[4] = {l4.x, l4.y, l4.z, l4.w}, dv4[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = g * 4 + e, i = i0 + rr + e;
        float sv = s[r];
        if (HAS_BIAS) sv = fmaf(bias[r], kAttnLog2e, sv);
        const bool valid = i < a.S && (!CAUSAL || j <= i);
        const float p = valid ? exp2f(sv - lv[e]) : 0.f;
        s[r] = p;
        dp[r] = p * (dp[r] - dv4[e]);
      }
    }
    f32_attn_weighted<DP>(do_s, s, lane, accv);
    f32_attn_weighted<DP>(q_s, dp, lane, acck);
  }
  if (!row_ok) return;
  f32_attn_store<T, DP>(dk + qkv_at(a, b, j, h), acck, scale, half, a.D, vec_qkv);
  f32_attn_store<T, DP>(dv + qkv_at(a, b, j, h), accv, 1.0f, half, a.D, vec_qkv);
}

}  // namespace mg
