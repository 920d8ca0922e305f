// Softmax cross-entropy forward / gradient / fused for one storage type T.  Included by
// one translation unit per dtype, which instantiates `CrossEntropyOps<T>`.
//
// Layout in HBM: logits, dense labels and dlogits are row-major (N, C); integer labels
// are (N) int32 or int64; per-row losses are (N) fp32 scratch; loss is one element of T.
//
// Gradient and fused kernels hold a whole row of logits in registers (chunks of VEC
// elements dealt round-robin to the TPR threads that share the row), so the logits are
// read from HBM once and dlogits written once.  The loss-only kernel streams the row
// once with an online softmax and keeps nothing.
#pragma once

#include <cstdlib>

#include "mg_device.h"
#include "mg_internal.h"
#include "mg_rows.h"

namespace mg {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

__device__ __forceinline__ float fast_exp2(float v) { return __builtin_amdgcn_exp2f(v); }

template <int TPR, int WG, int K>
__device__ __forceinline__ void row_allreduce_max(float (&v)[K], float* slots, int& phase) {
  if constexpr (TPR == 16) {
    // four rows side by side in a wave, each on one row of 16 lanes
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = row16_allreduce<MaxOp>(v[k]);
  } else if constexpr (TPR == kWave) {
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = wave_max(v[k]);
  } else {
    static_assert(TPR == WG, "a row is shared by sixteen lanes, one wave or the whole workgroup");
    block_allreduce<MaxOp, WG / kWave, K>(v, slots, phase);
    phase ^= 1;
  }
}

__device__ __forceinline__ int64_t load_id(const void* ids, int64_t row, bool id64) {
  return id64 ? static_cast<const int64_t*>(ids)[row] : static_cast<int64_t>(static_cast<const int32_t*>(ids)[row]);
}

// ------------------------------------------------------------------------------------
// Gradient (and optionally loss) with the row resident in registers.
//   labels: dense rows of T when DENSE, else N integer ids (int64 when id64).
//   rowloss: per-row loss term -sum(label * log_softmax) / N, or nullptr to skip.
//   upstream: one element of T, or nullptr for 1.
// ------------------------------------------------------------------------------------

template <typename T, int VEC, int TPR, int VPT, int WG, bool DENSE>
__global__ __launch_bounds__(WG, (TPR == 256 && VPT * VEC > 128) ? 2 : 1) void ce_rows_kernel(
    const T* __restrict__ logits, const void* __restrict__ labels, const T* __restrict__ upstream,
    float* __restrict__ rowloss, T* __restrict__ dlogits, int64_t N, int C, int id64) {
  constexpr int RPW = WG / TPR;
  using Tile = RowTile<T, VEC, TPR, VPT>;
  __shared__ float slots[2 * (WG / kWave)];
  int t, sub;
  row_thread<TPR, WG>(t, sub);
  int phase = 0;
  const float inv_rows = 1.0f / static_cast<float>(N);
  const float scale = (upstream != nullptr ? to_float(upstream[0]) : 1.0f) * inv_rows;

  // One row per TPR threads and no row loop: a loop would let the compiler start the next
  // row's loads before this row's stores and double the register footprint.
  {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * RPW + sub;
    if (row >= N) return;  // per 16-lane row, per wave or per workgroup (RPW == 1); no barrier follows for TPR <= 64
    const T* xr = logits + row * C;
    Tile x;
    x.load(xr, t, C);

    // Padding chunks hold zeros: mask them to -inf for the max and skip them in the sums.
    const int nfull = Tile::full_chunks(C);
    float m[1] = {-INFINITY};
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      if (i < nfull) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) m[0] = fmaxf(m[0], x.v[i][e]);
      } else if (i == nfull) {
        const bool valid = Tile::col(i, t) < C;
#pragma unroll
        for (int e = 0; e < VEC; ++e) m[0] = fmaxf(m[0], valid ? x.v[i][e] : -INFINITY);
      }
    }
    row_allreduce_max<TPR, WG, 1>(m, slots, phase);
    const float m2 = m[0] * kLog2e;
    T* out_row = dlogits + row * C;

    if constexpr (DENSE) {
      float s[1] = {0.f};
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        if (i < nfull) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) s[0] += fast_exp2(fmaf(x.v[i][e], kLog2e, -m2));
        } else if (i == nfull) {
          const bool valid = Tile::col(i, t) < C;
#pragma unroll
          for (int e = 0; e < VEC; ++e) s[0] += valid ? fast_exp2(fmaf(x.v[i][e], kLog2e, -m2)) : 0.f;
        }
      }
      row_allreduce_sum<TPR, WG, 1>(s, slots, phase);
      // softmax = exp(x - lse), formed directly from the log-sum-exp so that the
      // exponentials of the previous pass need not stay live next to the logits.
      const float shift = m[0] + logf(s[0]);
      const float shift2 = shift * kLog2e;
      const T* yr = static_cast<const T*>(labels) + row * C;
      float acc[1] = {0.f};
      const unsigned lane_off = static_cast<unsigned>(t) * VEC;
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        if (i < nfull || (i == nfull && Tile::col(i, t) < C)) {
          float y[VEC], out[VEC];
          VecIO<T, VEC>::load(yr + i * (TPR * VEC) + lane_off, y);
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            acc[0] += (x.v[i][e] - shift) * y[e];
            out[e] = (fast_exp2(fmaf(x.v[i][e], kLog2e, -shift2)) - y[e]) * scale;
          }
          VecIO<T, VEC>::store(out_row + i * (TPR * VEC) + lane_off, out);
        }
      }
      if (rowloss != nullptr) {
        row_allreduce_sum<TPR, WG, 1>(acc, slots, phase);
        if (t == 0) rowloss[row] = -acc[0] * inv_rows;
      }
    } else {
      // Integer labels: the exponentials replace the logits in registers, the gradient is
      // one multiply per element, and the single "- 1" at the label column is patched by
      // its owner thread with a scalar store issued after its vector stores (same thread,
      // same address: program order holds).
      float s[1] = {0.f};
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        if (i < nfull) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            x.v[i][e] = fast_exp2(fmaf(x.v[i][e], kLog2e, -m2));
            s[0] += x.v[i][e];
          }
        } else if (i == nfull) {
          const bool valid = Tile::col(i, t) < C;
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            x.v[i][e] = fast_exp2(fmaf(x.v[i][e], kLog2e, -m2));
            s[0] += valid ? x.v[i][e] : 0.f;
          }
        }
      }
      row_allreduce_sum<TPR, WG, 1>(s, slots, phase);
      const float k = scale / s[0];
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        if (i <= nfull) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) x.v[i][e] *= k;
        }
      }
      x.store(out_row, t, C);
      const int64_t id = load_id(labels, row, id64 != 0);
      const bool id_ok = id >= 0 && id < C;
      const bool owner = id_ok && (static_cast<int>(id) / VEC) % TPR == t;
      if (owner) {
        const float xl = to_float(xr[id]);
        const float lp = xl - m[0] - logf(s[0]);  // log softmax at the label
        out_row[id] = from_float<T>((fast_exp2(fmaf(xl, kLog2e, -m2)) / s[0] - 1.0f) * scale);
        if (rowloss != nullptr) rowloss[row] = -lp * inv_rows;
      }
      // An id outside [0, C) selects no column: the row's loss term is flagged NaN.
      if (rowloss != nullptr && !id_ok && t == 0) rowloss[row] = NAN;
    }
  }
}

// Integer labels, 16-bit logits, rows of thousands of columns: the row stays in
// registers as loaded (eight 16-bit values per 128-bit register quad) and is unpacked in each of
// its three passes (maximum, sum of exponentials, gradient), so a thread holds VPT * 4 registers
// for VPT * 8 columns instead of VPT * 8: 200 fp32 values per thread next to the 100 registers
// they were loaded into spill (656 bytes per lane at 50304 columns: 1.36 TB/s).  The second
// exponential per element is free in a kernel that waits for memory.  The arithmetic per element
// is that of ce_rows_kernel, so are the bits.  One row per workgroup.
template <typename T, int TPR, int VPT>
__global__ __launch_bounds__(TPR, TPR <= 256 ? (VPT > 16 ? 3 : 4) : (TPR <= 512 ? 2 : 1)) void ce_rows_packed_kernel(
    const T* __restrict__ logits, const void* __restrict__ labels, const T* __restrict__ upstream,
    float* __restrict__ rowloss, T* __restrict__ dlogits, int64_t N, int C, int id64) {
  static_assert(sizeof(T) == 2, "16-bit element types");
  constexpr int VEC = 8;
  __shared__ float slots[2 * (TPR / kWave)];
  const int t = threadIdx.x;
  int phase = 0;
  const float inv_rows = 1.0f / static_cast<float>(N);
  const float scale = (upstream != nullptr ? to_float(upstream[0]) : 1.0f) * inv_rows;
  const int64_t row = blockIdx.x;
  const T* xr = logits + row * C;
  T* out_row = dlogits + row * C;
  const int nfull = (C / VEC) / TPR;  // chunk indices below it exist for every thread
  const bool tail = (nfull * TPR + t) * VEC < C;  // this thread's chunk `nfull` exists

  uint4 raw[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    raw[i] = make_uint4(0, 0, 0, 0);
    if (i < nfull || (i == nfull && tail)) raw[i] = *reinterpret_cast<const uint4*>(xr + (i * TPR + t) * VEC);
  }
  float m[1] = {-INFINITY};
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if (i < nfull || (i == nfull && tail)) {
      float x[VEC];
      VecIO<T, VEC>::load(reinterpret_cast<const T*>(&raw[i]), x);
#pragma unroll
      for (int e = 0; e < VEC; ++e) m[0] = fmaxf(m[0], x[e]);
    }
  }
  row_allreduce_max<TPR, TPR, 1>(m, slots, phase);
  const float m2 = m[0] * kLog2e;
  // Between the passes the packed registers are made opaque to the compiler, which would
  // otherwise keep the unpacked values of one pass for the next.
  auto forget = [&]() {
#pragma unroll
    for (int i = 0; i < VPT; ++i) asm volatile("" : "+v"(raw[i].x), "+v"(raw[i].y), "+v"(raw[i].z), "+v"(raw[i].w));
  };
  forget();
  float s[1] = {0.f};
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if (i < nfull || (i == nfull && tail)) {
      float x[VEC];
      VecIO<T, VEC>::load(reinterpret_cast<const T*>(&raw[i]), x);
#pragma unroll
      for (int e = 0; e < VEC; ++e) s[0] += fast_exp2(fmaf(x[e], kLog2e, -m2));
    }
  }
  row_allreduce_sum<TPR, TPR, 1>(s, slots, phase);
  const float k = scale / s[0];
  forget();
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if (i < nfull || (i == nfull && tail)) {
      float x[VEC];
      VecIO<T, VEC>::load(reinterpret_cast<const T*>(&raw[i]), x);
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[e] = fast_exp2(fmaf(x[e], kLog2e, -m2)) * k;
      VecIO<T, VEC>::store(out_row + (i * TPR + t) * VEC, x);
    }
  }
  // the "- 1" at the label column: a scalar store by the thread that owns the column, after its
  // vector stores (same thread, same address: program order holds)
  const int64_t id = load_id(labels, row, id64 != 0);
  const bool id_ok = id >= 0 && id < C;
  if (id_ok && (static_cast<int>(id) / VEC) % TPR == t) {
    const float xl = to_float(xr[id]);
    const float lp = xl - m[0] - logf(s[0]);  // log softmax at the label
    out_row[id] = from_float<T>((fast_exp2(fmaf(xl, kLog2e, -m2)) / s[0] - 1.0f) * scale);
    if (rowloss != nullptr) rowloss[row] = -lp * inv_rows;
  }
  // An id outside [0, C) selects no column: the row's loss term is flagged NaN.
  if (rowloss != nullptr && !id_ok && t == 0) rowloss[row] = NAN;
}

// ------------------------------------------------------------------------------------
// Streaming kernels: any C, any alignment.  One workgroup per row.
// ------------------------------------------------------------------------------------

// Online (max, sum-exp) over the elements a thread visits, merged across the workgroup.  ONCE: the
// row is not read again by this kernel, so its loads go past the caches.
template <typename T, int VEC, int WG, bool ONCE = false>
__device__ __forceinline__ void stream_max_sum(const T* __restrict__ xr, int64_t C, float* slots, int& phase, float& m_out,
                                               float& s_out) {
  auto fetch = [](const T* p, float (&v)[VEC]) {
    if constexpr (ONCE) VecIO<T, VEC>::load_stream(p, v);
    else VecIO<T, VEC>::load(p, v);
  };
  float m = -INFINITY, s = 0.f;
  constexpr int U = 4;  // chunks in flight per thread: the loop is bound by memory-level parallelism
  const int64_t step = static_cast<int64_t>(WG) * VEC;
  int64_t c = static_cast<int64_t>(threadIdx.x) * VEC;
  for (; c + (U - 1) * step < C; c += U * step) {
    float v[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) fetch(xr + c + u * step, v[u]);
    float cm = v[0][0];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int e = 0; e < VEC; ++e) cm = fmaxf(cm, v[u][e]);
    if (cm > m) {
      s *= fast_exp2((m - cm) * kLog2e);  // exp2(-inf) == 0 on the first chunk
      m = cm;
    }
    const float m2 = m * kLog2e;
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int e = 0; e < VEC; ++e) s += fast_exp2(fmaf(v[u][e], kLog2e, -m2));
  }
  for (; c < C; c += step) {
    float v[VEC];
    fetch(xr + c, v);
    float cm = v[0];
#pragma unroll
    for (int e = 1; e < VEC; ++e) cm = fmaxf(cm, v[e]);
    if (cm > m) {
      s *= fast_exp2((m - cm) * kLog2e);
      m = cm;
    }
    const float m2 = m * kLog2e;
#pragma unroll
    for (int e = 0; e < VEC; ++e) s += fast_exp2(fmaf(v[e], kLog2e, -m2));
  }
  float mm[1] = {m};
  block_allreduce<MaxOp, WG / kWave, 1>(mm, slots, phase);
  phase ^= 1;
  // Threads that saw nothing have m == -inf and s == 0; (m - mm) would be nan only if the
  // whole row were empty, which C > 0 excludes.
  float ss[1] = {m == -INFINITY ? 0.f : s * fast_exp2((m - mm[0]) * kLog2e)};
  block_allreduce<SumOp, WG / kWave, 1>(ss, slots, phase);
  phase ^= 1;
  m_out = mm[0];
  s_out = ss[0];
}

// Loss only.  Dense: sum(label * (x - lse)) = sum(label * x) - lse * sum(label), so one
// pass over logits and labels suffices.
// ONCE: the logits (and dense labels) are larger than the memory-side cache can hold, so they are
// read past the caches (1.65 GB of logits: 266 -> 238 us, 6.9 TB/s; smaller tensors may still be
// cached from the kernel that wrote them and keep the plain loads).
template <typename T, int VEC, int WG, bool DENSE, bool ONCE = false>
__global__ __launch_bounds__(WG) void ce_fwd_stream_kernel(const T* __restrict__ logits, const void* __restrict__ labels,
                                                           float* __restrict__ rowloss, int64_t N, int64_t C, int id64) {
  __shared__ float slots[2 * 2 * (WG / kWave)];
  int phase = 0;
  const int64_t row = blockIdx.x;
  if (row >= N) return;
  const T* xr = logits + row * C;
  float m, s;
  const float inv_rows = 1.0f / static_cast<float>(N);
  if constexpr (DENSE) {
    const T* yr = static_cast<const T*>(labels) + row * C;
    float dot[2] = {0.f, 0.f};  // sum(label * x), sum(label)
    float tm = -INFINITY, ts = 0.f;
    for (int64_t c = static_cast<int64_t>(threadIdx.x) * VEC; c < C; c += static_cast<int64_t>(WG) * VEC) {
      float v[VEC], y[VEC];
      if constexpr (ONCE) {
        VecIO<T, VEC>::load_stream(xr + c, v);
        VecIO<T, VEC>::load_stream(yr + c, y);
      } else {
        VecIO<T, VEC>::load(xr + c, v);
        VecIO<T, VEC>::load(yr + c, y);
      }
      float cm = v[0];
#pragma unroll
      for (int e = 1; e < VEC; ++e) cm = fmaxf(cm, v[e]);
      if (cm > tm) {
        ts *= fast_exp2((tm - cm) * kLog2e);
        tm = cm;
      }
      const float m2 = tm * kLog2e;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        ts += fast_exp2(fmaf(v[e], kLog2e, -m2));
        dot[0] += v[e] * y[e];
        dot[1] += y[e];
      }
    }
    float mm[1] = {tm};
    block_allreduce<MaxOp, WG / kWave, 1>(mm, slots, phase);
    phase ^= 1;
    float red[3] = {tm == -INFINITY ? 0.f : ts * fast_exp2((tm - mm[0]) * kLog2e), dot[0], dot[1]};
    __shared__ float slots3[2 * 3 * (WG / kWave)];
    block_allreduce<SumOp, WG / kWave, 3>(red, slots3, 0);
    m = mm[0];
    s = red[0];
    if (threadIdx.x == 0) rowloss[row] = -(red[1] - (m + logf(s)) * red[2]) * inv_rows;
  } else {
    stream_max_sum<T, VEC, WG, ONCE>(xr, C, slots, phase, m, s);
    if (threadIdx.x == 0) {
      const int64_t id = load_id(labels, row, id64 != 0);
      rowloss[row] = (id < 0 || id >= C) ? NAN : -(to_float(xr[id]) - (m + logf(s))) * inv_rows;
    }
  }
}

// Gradient (and optionally loss) for rows too wide for registers: two passes.
template <typename T, int VEC, int WG, bool DENSE>
__global__ __launch_bounds__(WG) void ce_grad_stream_kernel(const T* __restrict__ logits, const void* __restrict__ labels,
                                                            const T* __restrict__ upstream, float* __restrict__ rowloss,
                                                            T* __restrict__ dlogits, int64_t N, int64_t C, int id64) {
  __shared__ float slots[2 * 2 * (WG / kWave)];
  int phase = 0;
  const int64_t row = blockIdx.x;
  if (row >= N) return;
  const T* xr = logits + row * C;
  T* out_row = dlogits + row * C;
  const float inv_rows = 1.0f / static_cast<float>(N);
  const float scale = (upstream != nullptr ? to_float(upstream[0]) : 1.0f) * inv_rows;
  float m, s;
  stream_max_sum<T, VEC, WG>(xr, C, slots, phase, m, s);
  const float m2 = m * kLog2e;
  const float inv_sum = 1.0f / s;
  const float shift = m + logf(s);
  const int64_t id = DENSE ? 0 : load_id(labels, row, id64 != 0);
  float acc[1] = {0.f};
  constexpr int U = DENSE ? 1 : 4;  // integer labels: four chunks in flight per thread
  const int64_t step = static_cast<int64_t>(WG) * VEC;
  int64_t c0 = static_cast<int64_t>(threadIdx.x) * VEC;
  if constexpr (!DENSE) {
    for (; c0 + (U - 1) * step < C; c0 += U * step) {
      float v[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) VecIO<T, VEC>::load(xr + c0 + u * step, v[u]);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t c = c0 + u * step;
        float out[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          float p = fast_exp2(fmaf(v[u][e], kLog2e, -m2)) * inv_sum;
          if (c + e == id) {
            p -= 1.0f;
            acc[0] += v[u][e] - shift;
          }
          out[e] = p * scale;
        }
        VecIO<T, VEC>::store(out_row + c, out);
      }
    }
  }
  for (int64_t c = c0; c < C; c += step) {
    float v[VEC], out[VEC];
    VecIO<T, VEC>::load(xr + c, v);
    if constexpr (DENSE) {
      float y[VEC];
      VecIO<T, VEC>::load(static_cast<const T*>(labels) + row * C + c, y);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        acc[0] += (v[e] - shift) * y[e];
        out[e] = (fast_exp2(fmaf(v[e], kLog2e, -m2)) * inv_sum - y[e]) * scale;
      }
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float p = fast_exp2(fmaf(v[e], kLog2e, -m2)) * inv_sum;
        if (c + e == id) {
          p -= 1.0f;
          acc[0] += v[e] - shift;
        }
        out[e] = p * scale;
      }
    }
    VecIO<T, VEC>::store(out_row + c, out);
  }
  if (rowloss != nullptr) {
    block_allreduce<SumOp, WG / kWave, 1>(acc, slots, phase);
    if (threadIdx.x == 0) rowloss[row] = (!DENSE && (id < 0 || id >= C)) ? NAN : -acc[0] * inv_rows;
  }
}

// ------------------------------------------------------------------------------------
// Strided views (rank <= 8): element offset from a flat index by div/mod over the shape,
// as the reference's strided kernels do (kernels/cross_entropy.mojo:80-152,244-307).
// ------------------------------------------------------------------------------------

__device__ __forceinline__ int64_t strided_offset(int64_t flat, const StridedView& v) {
  int64_t off = 0;
  for (int d = v.rank - 1; d >= 0; --d) {
    off += (flat % v.shape[d]) * v.stride[d];
    flat /= v.shape[d];
  }
  return off;
}

template <typename T, int WG, bool WANT_GRAD>
__global__ __launch_bounds__(WG) void ce_strided_kernel(const T* __restrict__ logits, const T* __restrict__ labels,
                                                        const T* __restrict__ upstream, float* __restrict__ rowloss,
                                                        T* __restrict__ dlogits, int64_t N, int64_t C, StridedView la,
                                                        StridedView lb) {
  __shared__ float slots[2 * (WG / kWave)];
  int phase = 0;
  const int64_t row = blockIdx.x;
  if (row >= N) return;
  const int64_t base = row * C;
  float m[1] = {-INFINITY};
  for (int64_t c = threadIdx.x; c < C; c += WG) m[0] = fmaxf(m[0], to_float(logits[strided_offset(base + c, la)]));
  block_allreduce<MaxOp, WG / kWave, 1>(m, slots, phase);
  phase ^= 1;
  const float m2 = m[0] * kLog2e;
  float s[1] = {0.f};
  for (int64_t c = threadIdx.x; c < C; c += WG)
    s[0] += fast_exp2(fmaf(to_float(logits[strided_offset(base + c, la)]), kLog2e, -m2));
  block_allreduce<SumOp, WG / kWave, 1>(s, slots, phase);
  phase ^= 1;
  const float inv_rows = 1.0f / static_cast<float>(N);
  if constexpr (WANT_GRAD) {
    const float inv_sum = 1.0f / s[0];
    const float scale = (upstream != nullptr ? to_float(upstream[0]) : 1.0f) * inv_rows;
    for (int64_t c = threadIdx.x; c < C; c += WG) {
      const float x = to_float(logits[strided_offset(base + c, la)]);
      const float y = to_float(labels[strided_offset(base + c, lb)]);
      dlogits[base + c] = from_float<T>((fast_exp2(fmaf(x, kLog2e, -m2)) * inv_sum - y) * scale);
    }
  } else {
    const float shift = m[0] + logf(s[0]);
    float acc[1] = {0.f};
    for (int64_t c = threadIdx.x; c < C; c += WG) {
      const float x = to_float(logits[strided_offset(base + c, la)]);
      const float y = to_float(labels[strided_offset(base + c, lb)]);
      acc[0] += (x - shift) * y;
    }
    block_allreduce<SumOp, WG / kWave, 1>(acc, slots, phase);
    if (threadIdx.x == 0) rowloss[row] = -acc[0] * inv_rows;
  }
}

// loss[0] = sum of the N per-row terms, one workgroup, fixed order (no atomics).
template <typename T>
__global__ __launch_bounds__(1024) void sum_rows_kernel(const float* __restrict__ rowloss, T* __restrict__ loss, int64_t N) {
  __shared__ float slots[2 * 16];
  float acc[1] = {0.f};
  for (int64_t i = threadIdx.x; i < N; i += 1024) acc[0] += rowloss[i];
  block_allreduce<SumOp, 16, 1>(acc, slots, 0);
  if (threadIdx.x == 0) loss[0] = from_float<T>(acc[0]);
}

// ------------------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------------------

template <typename T>
struct CrossEntropyOps {
  static constexpr int WIDE = WideVec<T>::value;
  struct Shape {
    int tpr, vpt;
  };

  // Thread layout for a row of `chunks` chunks held in registers; false if too wide.
  static bool pick_shape(int64_t chunks, bool wide, Shape* s) {
    // Rows of up to 80 unaligned elements (a 65-symbol vocabulary): sixteen lanes per row, four
    // rows per wave; one wave per row left most lanes idle and a latency per 130 bytes.
    if (!wide && chunks <= 80 && env_int("MOGRAD_HIP_CE_NARROW", 1) != 0) *s = {16, 5};
    else if (chunks <= 64) *s = {64, 1};
    else if (chunks <= 128) *s = {64, 2};
    else if (chunks <= 256) *s = {64, 4};
    else if (chunks <= 1024) *s = {256, 4};
    else if (chunks <= 2048) *s = {512, 4};
    else if (chunks <= 4096) *s = {512, 8};
    else if (WIDE == 8 && wide && chunks <= 6400) *s = {256, 25};  // 16-bit rows up to 51200 columns: see below
    else if (chunks <= 8192) *s = {512, 16};
    else if (WIDE == 4 && wide && chunks <= 12800) *s = {256, 50};
    else if (wide && chunks <= 16384) *s = {1024, 16};
    else return false;
    // Rows of about 50k columns (8193..12800 fp32 chunks, 4097..6400 16-bit chunks: 200
    // values per thread either way): 256 threads x 50 (fp32) or x 25 (16-bit) chunks by
    // default, which leaves room for two workgroups per CU so that one row's arithmetic
    // overlaps the other's memory traffic.  MOGRAD_HIP_CE_WIDE_ROW=512|1024 selects the
    // 512 x 25 or 1024 x 13 layout instead (tuning aid).
    if (WIDE == 4 && wide && chunks > 8192 && chunks <= 12800) {
      const int pick = env_int("MOGRAD_HIP_CE_WIDE_ROW", 256);
      if (pick == 512) *s = {512, 25};
      if (pick == 1024) *s = {1024, 13};
    }
    return true;
  }

  static bool can_vectorise(int64_t C, std::initializer_list<const void*> ptrs) {
    if (WIDE == 1 || C % WIDE != 0) return false;
    for (const void* p : ptrs)
      if (p != nullptr && !aligned16(p)) return false;
    return true;
  }

  static unsigned row_grid(int64_t N, int rpw) {
    return static_cast<unsigned>(ceil_div(N, rpw));
  }

  template <int VEC, int TPR, int VPT, bool DENSE>
  static int launch_rows(const T* logits, const void* labels, const T* upstream, float* rowloss, T* dlogits, int64_t N,
                         int64_t C, int id64, hipStream_t stream) {
    constexpr int WG = TPR <= 64 ? 256 : TPR;
    hipLaunchKernelGGL((ce_rows_kernel<T, VEC, TPR, VPT, WG, DENSE>), dim3(row_grid(N, WG / TPR)), dim3(WG), 0, stream,
                       logits, labels, upstream, rowloss, dlogits, N, static_cast<int>(C), id64);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }

  template <int VEC, bool DENSE>
  static int dispatch_rows(Shape s, const T* logits, const void* labels, const T* upstream, float* rowloss, T* dlogits,
                           int64_t N, int64_t C, int id64, hipStream_t stream) {
#define MG_CE_CASE(TPR_, VPT_)        \
  if (s.tpr == TPR_ && s.vpt == VPT_) \
  return launch_rows<VEC, TPR_, VPT_, DENSE>(logits, labels, upstream, rowloss, dlogits, N, C, id64, stream)
    MG_CE_CASE(16, 5);
    MG_CE_CASE(64, 1);
    MG_CE_CASE(64, 2);
    MG_CE_CASE(64, 4);
    MG_CE_CASE(256, 4);
    MG_CE_CASE(512, 4);
    MG_CE_CASE(512, 8);
    MG_CE_CASE(512, 16);
    if constexpr (VEC == 8) {
      MG_CE_CASE(256, 25);
    }
    if constexpr (VEC > 1) {
      MG_CE_CASE(256, 50);
      MG_CE_CASE(512, 25);
      MG_CE_CASE(1024, 13);
      MG_CE_CASE(1024, 16);
    }
#undef MG_CE_CASE
    return fail(MG_ERR_UNSUPPORTED, "cross_entropy: no kernel for row shape (%d, %d)", s.tpr, s.vpt);
  }

  static int finish_loss(const float* rowloss, T* loss, int64_t N, hipStream_t stream) {
    hipLaunchKernelGGL((sum_rows_kernel<T>), dim3(1), dim3(1024), 0, stream, rowloss, loss, N);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }

  // Gradient and/or loss.  `loss` and `dlogits` may each be null (not both).
  // `rowloss_ext`, when not null, is a buffer of at least N floats that takes the per-row
  // loss terms instead of a block from the pool (the entry point that allocates nothing).
  template <bool DENSE>
  static int run(const void* logits_, const void* labels, const void* upstream_, void* loss_, void* dlogits_, int64_t N,
                 int64_t C, int id64, hipStream_t stream, float* rowloss_ext = nullptr) {
    const T* logits = static_cast<const T*>(logits_);
    const T* upstream = static_cast<const T*>(upstream_);
    T* loss = static_cast<T*>(loss_);
    T* dlogits = static_cast<T*>(dlogits_);
    Scratch rowloss_buf;
    float* rowloss = nullptr;
    if (loss != nullptr && rowloss_ext != nullptr) {
      rowloss = rowloss_ext;
    } else if (loss != nullptr) {
      MG_TRY(rowloss_buf.take(N * static_cast<int64_t>(sizeof(float))));
      rowloss = rowloss_buf.as<float>();
    }
    const bool wide = can_vectorise(C, {logits, DENSE ? labels : nullptr, dlogits});
    constexpr int SWG = 1024;
    if (dlogits == nullptr) {
      // larger than the 256 MB memory-side cache: read once, past the caches
      const bool once = N * C * static_cast<int64_t>(sizeof(T)) >= (int64_t{256} << 20);
      if (wide && once)
        hipLaunchKernelGGL((ce_fwd_stream_kernel<T, WIDE, SWG, DENSE, true>), dim3(static_cast<unsigned>(N)), dim3(SWG), 0,
                           stream, logits, labels, rowloss, N, C, id64);
      else if (wide)
        hipLaunchKernelGGL((ce_fwd_stream_kernel<T, WIDE, SWG, DENSE>), dim3(static_cast<unsigned>(N)), dim3(SWG), 0,
                           stream, logits, labels, rowloss, N, C, id64);
      else
        hipLaunchKernelGGL((ce_fwd_stream_kernel<T, 1, 256, DENSE>), dim3(static_cast<unsigned>(N)), dim3(256), 0,
                           stream, logits, labels, rowloss, N, C, id64);
      MG_LAUNCH_CHECK();
      return finish_loss(rowloss, loss, N, stream);
    }
    Shape s;
    if constexpr (sizeof(T) == 2 && !DENSE) {
      // 16-bit rows of more than 512 chunks (4096 columns) with integer labels: the packed row
      // kernel ((8192, 50304) bf16 1220 -> 344 us, (16384, 16392) 415 -> 209 us, (65536, 4104)
      // 275 -> 205 us, (32768, 8192) 197 us either way).  MOGRAD_HIP_CE_PACKED=0: the fp32 tiles.
      const int64_t chunks = C / WIDE;
      if (wide && chunks > 512 && chunks <= 16384 && dlogits != nullptr && env_int("MOGRAD_HIP_CE_PACKED", 1) != 0) {
        const unsigned grid = static_cast<unsigned>(N);
        const int Ci = static_cast<int>(C);
        if (chunks <= 1024)
          hipLaunchKernelGGL((ce_rows_packed_kernel<T, 256, 4>), dim3(grid), dim3(256), 0, stream, logits, labels, upstream,
                             rowloss, dlogits, N, Ci, id64);
        else if (chunks <= 2048)
          hipLaunchKernelGGL((ce_rows_packed_kernel<T, 256, 8>), dim3(grid), dim3(256), 0, stream, logits, labels, upstream,
                             rowloss, dlogits, N, Ci, id64);
        else if (chunks <= 4096)
          hipLaunchKernelGGL((ce_rows_packed_kernel<T, 256, 16>), dim3(grid), dim3(256), 0, stream, logits, labels, upstream,
                             rowloss, dlogits, N, Ci, id64);
        else if (chunks <= 6400)
          hipLaunchKernelGGL((ce_rows_packed_kernel<T, 256, 25>), dim3(grid), dim3(256), 0, stream, logits, labels, upstream,
                             rowloss, dlogits, N, Ci, id64);
        else if (chunks <= 12800)
          hipLaunchKernelGGL((ce_rows_packed_kernel<T, 512, 25>), dim3(grid), dim3(512), 0, stream, logits, labels, upstream,
                             rowloss, dlogits, N, Ci, id64);
        else
          hipLaunchKernelGGL((ce_rows_packed_kernel<T, 1024, 16>), dim3(grid), dim3(1024), 0, stream, logits, labels,
                             upstream, rowloss, dlogits, N, Ci, id64);
        MG_LAUNCH_CHECK();
        if (loss != nullptr) return finish_loss(rowloss, loss, N, stream);
        return MG_OK;
      }
    }
    if (wide && pick_shape(C / WIDE, true, &s)) {
      MG_TRY((dispatch_rows<WIDE, DENSE>(s, logits, labels, upstream, rowloss, dlogits, N, C, id64, stream)));
    } else if (!wide && pick_shape(C, false, &s)) {
      MG_TRY((dispatch_rows<1, DENSE>(s, logits, labels, upstream, rowloss, dlogits, N, C, id64, stream)));
    } else {
      if (wide)
        hipLaunchKernelGGL((ce_grad_stream_kernel<T, WIDE, SWG, DENSE>), dim3(static_cast<unsigned>(N)), dim3(SWG), 0,
                           stream, logits, labels, upstream, rowloss, dlogits, N, C, id64);
      else
        hipLaunchKernelGGL((ce_grad_stream_kernel<T, 1, SWG, DENSE>), dim3(static_cast<unsigned>(N)), dim3(SWG), 0,
                           stream, logits, labels, upstream, rowloss, dlogits, N, C, id64);
      MG_LAUNCH_CHECK();
    }
    if (loss != nullptr) return finish_loss(rowloss, loss, N, stream);
    return MG_OK;
  }

  static int run_strided(const void* logits_, const void* labels_, const void* upstream_, void* loss_, void* dlogits_,
                         int64_t N, int64_t C, const StridedView& la, const StridedView& lb, hipStream_t stream) {
    const T* logits = static_cast<const T*>(logits_);
    const T* labels = static_cast<const T*>(labels_);
    const T* upstream = static_cast<const T*>(upstream_);
    T* loss = static_cast<T*>(loss_);
    T* dlogits = static_cast<T*>(dlogits_);
    if (dlogits != nullptr) {
      hipLaunchKernelGGL((ce_strided_kernel<T, 256, true>), dim3(static_cast<unsigned>(N)), dim3(256), 0, stream, logits,
                         labels, upstream, nullptr, dlogits, N, C, la, lb);
      MG_LAUNCH_CHECK();
      return MG_OK;
    }
    Scratch rowloss;
    MG_TRY(rowloss.take(N * static_cast<int64_t>(sizeof(float))));
    hipLaunchKernelGGL((ce_strided_kernel<T, 256, false>), dim3(static_cast<unsigned>(N)), dim3(256), 0, stream, logits,
                       labels, upstream, rowloss.as<float>(), dlogits, N, C, la, lb);
    MG_LAUNCH_CHECK();
    return finish_loss(rowloss.as<float>(), loss, N, stream);
  }
};

}  // namespace mg

// Defines the per-dtype entry points that cross_entropy.hip dispatches to.
#define MG_DEFINE_CROSS_ENTROPY(T, SUFFIX)                                                                          \
  namespace mg {                                                                                                    \
  int ce_run_##SUFFIX(bool dense, const void* logits, const void* labels, const void* upstream, void* loss,         \
                      void* dlogits, int64_t N, int64_t C, int id64, hipStream_t stream, float* rowloss_ext) {      \
    if (dense)                                                                                                      \
      return CrossEntropyOps<T>::template run<true>(logits, labels, upstream, loss, dlogits, N, C, id64, stream,    \
                                                    rowloss_ext);                                                   \
    return CrossEntropyOps<T>::template run<false>(logits, labels, upstream, loss, dlogits, N, C, id64, stream,     \
                                                   rowloss_ext);                                                    \
  }                                                                                                                 \
  int ce_run_strided_##SUFFIX(const void* logits, const void* labels, const void* upstream, void* loss,             \
                              void* dlogits, int64_t N, int64_t C, const StridedView& la, const StridedView& lb,    \
                              hipStream_t stream) {                                                                 \
    return CrossEntropyOps<T>::run_strided(logits, labels, upstream, loss, dlogits, N, C, la, lb, stream);          \
  }                                                                                                                 \
  }
