// LayerNorm forward and backward for one storage type T.  Included by one translation
// unit per dtype (layer_norm_f32.hip, ...), which instantiates `LayerNormOps<T>`.
//
// Layout in HBM: x, dy, y, dx are row-major (rows, cols); gamma, beta, dgamma, dbeta are
// (cols); mean, rstd are (rows) fp32.  Partial column sums are fp32 (groups, cols).
//
// Row kernels keep a whole row in registers: a row is split into chunks of VEC elements,
// chunk i of a row belongs to thread (i % TPR) as its (i / TPR)-th chunk, so a wave reads
// 64 consecutive 16-byte chunks per load instruction.  TPR threads share one row; a
// workgroup of WG threads works on WG/TPR rows at a time.  x and dy are read from HBM
// exactly once and dx written once.
#pragma once

#include "mg_device.h"
#include "mg_internal.h"
#include "mg_rows.h"

namespace mg {

// Mean and rstd of the row held in `x` (shifted sums: the shift is the row's first
// element, which keeps E[d^2] - E[d]^2 free of cancellation for rows with a large mean).
template <typename T, int VEC, int TPR, int VPT, int WG>
__device__ __forceinline__ void row_stats(const RowTile<T, VEC, TPR, VPT>& x, float shift, int t, int cols,
                                          float eps, float* slots, int& phase, float& mu, float& rstd) {
  float s[2] = {0.f, 0.f};
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if (RowTile<T, VEC, TPR, VPT>::col(i, t) < cols) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float d = x.v[i][e] - shift;
        s[0] += d;
        s[1] += d * d;
      }
    }
  }
  row_allreduce_sum<TPR, WG, 2>(s, slots, phase);
  const float inv_n = 1.0f / static_cast<float>(cols);
  const float md = s[0] * inv_n;
  const float var = fmaxf(s[1] * inv_n - md * md, 0.f);
  mu = shift + md;
  rstd = rsqrtf(var + eps);
}

// ------------------------------------------------------------------------------------
// Forward
// ------------------------------------------------------------------------------------

template <typename T, int VEC, int TPR, int VPT, int WG>
__global__ __launch_bounds__(WG) void ln_fwd_rows_kernel(const T* __restrict__ x, const T* __restrict__ gamma,
                                                         const T* __restrict__ beta, T* __restrict__ y,
                                                         float* __restrict__ mean_out, float* __restrict__ rstd_out,
                                                         int64_t rows, int cols, float eps) {
  constexpr int RPW = WG / TPR;
  __shared__ float slots[2 * 2 * (WG / kWave)];
  int t, sub;
  row_thread<TPR, WG>(t, sub);
  int phase = 0;

  RowTile<T, VEC, TPR, VPT> g, b;
  g.load(gamma, t, cols);
  b.load(beta, t, cols);

  for (int64_t row0 = static_cast<int64_t>(blockIdx.x) * RPW; row0 < rows; row0 += static_cast<int64_t>(gridDim.x) * RPW) {
    const int64_t row = row0 + sub;
    if (row >= rows) continue;  // uniform per row of 16 lanes (TPR == 16), per wave (64) or per workgroup (RPW == 1)
    RowTile<T, VEC, TPR, VPT> xv;
    xv.load(x + row * cols, t, cols);
    const float shift = to_float(x[row * cols]);
    float mu, rstd;
    row_stats<T, VEC, TPR, VPT, WG>(xv, shift, t, cols, eps, slots, phase, mu, rstd);
#pragma unroll
    for (int i = 0; i < VPT; ++i)
#pragma unroll
      for (int e = 0; e < VEC; ++e) xv.v[i][e] = (xv.v[i][e] - mu) * rstd * g.v[i][e] + b.v[i][e];
    xv.store_stream(y + row * cols, t, cols);
    if (mean_out != nullptr && t == 0) {
      mean_out[row] = mu;
      rstd_out[row] = rstd;
    }
  }
}

// Forward fallback for rows too wide to hold in registers: one workgroup per row,
// two streaming passes.
template <typename T, int WG>
__global__ __launch_bounds__(WG) void ln_fwd_stream_kernel(const T* __restrict__ x, const T* __restrict__ gamma,
                                                           const T* __restrict__ beta, T* __restrict__ y,
                                                           float* __restrict__ mean_out, float* __restrict__ rstd_out,
                                                           int64_t rows, int64_t cols, float eps) {
  __shared__ float slots[2 * 2 * (WG / kWave)];
  const int64_t row = blockIdx.x;
  if (row >= rows) return;
  const T* xr = x + row * cols;
  const float shift = to_float(xr[0]);
  float s[2] = {0.f, 0.f};
  for (int64_t c = threadIdx.x; c < cols; c += WG) {
    const float d = to_float(xr[c]) - shift;
    s[0] += d;
    s[1] += d * d;
  }
  block_allreduce<SumOp, WG / kWave, 2>(s, slots, 0);
  const float inv_n = 1.0f / static_cast<float>(cols);
  const float md = s[0] * inv_n;
  const float mu = shift + md;
  const float rstd = rsqrtf(fmaxf(s[1] * inv_n - md * md, 0.f) + eps);
  for (int64_t c = threadIdx.x; c < cols; c += WG)
    y[row * cols + c] = from_float<T>((to_float(xr[c]) - mu) * rstd * to_float(gamma[c]) + to_float(beta[c]));
  if (mean_out != nullptr && threadIdx.x == 0) {
    mean_out[row] = mu;
    rstd_out[row] = rstd;
  }
}

// ------------------------------------------------------------------------------------
// Backward, stage 1: dx per row, and per-workgroup partial sums of dy*xhat and dy.
// Workgroup g owns rows [g*rows_per_group, (g+1)*rows_per_group).
// ------------------------------------------------------------------------------------

template <typename T, int VEC, int TPR, int VPT, int WG, bool HAS_STATS>
__global__ __launch_bounds__(WG) void ln_bwd_rows_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                         const T* __restrict__ gamma, const float* __restrict__ mean_in,
                                                         const float* __restrict__ rstd_in, const T* residual,
                                                         T* dx, float* __restrict__ part_g,
                                                         float* __restrict__ part_b, int64_t rows, int cols, float eps,
                                                         int64_t rows_per_group, int64_t row_step) {
  constexpr int RPW = WG / TPR;
  constexpr int NW = WG / kWave;
  constexpr int TILE_COLS = VPT * TPR * VEC;
  __shared__ float slots[2 * 4 * NW];
  // Only used to combine the RPW row slots of one workgroup at the end: one set of column sums
  // per wave (rows narrower than a wave are first added across the wave's rows of lanes).
  constexpr int SETS = TPR < kWave ? NW : RPW;
  __shared__ float combine[RPW > 1 ? SETS * TILE_COLS : 1];

  int t, sub;
  row_thread<TPR, WG>(t, sub);
  int phase = 0;

  RowTile<T, VEC, TPR, VPT> g, acc_g, acc_b;
  g.load(gamma, t, cols);
  acc_g.zero();
  acc_b.zero();

  // row_step == RPW: the group's rows are consecutive; otherwise its rows lie row_step apart
  // (the groups interleaved, every trip of the loop reading one contiguous band of the matrix).
  const int64_t r_begin = row_step == RPW ? static_cast<int64_t>(blockIdx.x) * rows_per_group
                                          : static_cast<int64_t>(blockIdx.x) * RPW;
  const int64_t r_end = row_step == RPW ? min(r_begin + rows_per_group, rows) : rows;
  const float inv_n = 1.0f / static_cast<float>(cols);

  // With narrow per-thread tiles the next row is fetched while this row is reduced;
  // wide tiles would spill, and rely on other resident workgroups to cover the latency.
  constexpr bool PREFETCH = VPT * VEC <= 8;
  // Rows that several waves share reduce through LDS with workgroup barriers, so when such
  // rows sit side by side in a workgroup every one of them makes every trip of the loop; a
  // row slot past the end of the group works on zeros and touches no memory.
  constexpr bool LOCKSTEP = TPR > kWave && RPW > 1;
  RowTile<T, VEC, TPR, VPT> xv, dyv, xn, dyn;
  int64_t row = r_begin + sub;
  // The row's scalars travel with its tile: the saved statistics, or the row's first element
  // (the shift of the one-pass sums), fetched a trip ahead like the tile itself.
  float sc0 = 0.f, sc1 = 0.f, sc0_n = 0.f, sc1_n = 0.f;
  auto load_scalars = [&](int64_t r, float& a, float& b) {
    if constexpr (HAS_STATS) {
      a = mean_in[r];
      b = rstd_in[r];
    } else {
      a = to_float(x[r * cols]);
    }
  };
  if (PREFETCH && row < r_end) {
    xv.load(x + row * cols, t, cols);
    dyv.load(dy + row * cols, t, cols);
    load_scalars(row, sc0, sc1);
  }
  for (; LOCKSTEP ? row - sub < r_end : row < r_end; row += row_step) {
    const bool active = !LOCKSTEP || row < r_end;
    if (LOCKSTEP && !active) {
      xv.zero();
      dyv.zero();
    }
    const int64_t next = row + row_step;
    if constexpr (PREFETCH) {
      if (next < r_end) {
        xn.load(x + next * cols, t, cols);
        dyn.load(dy + next * cols, t, cols);
        load_scalars(next, sc0_n, sc1_n);
      }
    } else if (active) {
      xv.load(x + row * cols, t, cols);
      dyv.load(dy + row * cols, t, cols);
      load_scalars(row, sc0, sc1);
    }
    float mu, rstd, c1, c2;
    if constexpr (HAS_STATS) {
      mu = active ? sc0 : 0.f;
      rstd = active ? sc1 : 0.f;
      // xhat replaces x; dy*gamma is formed on the fly.  Columns past `cols` hold zeros in
      // dy and gamma, so they add nothing to the sums.
      float s[2] = {0.f, 0.f};
#pragma unroll
      for (int i = 0; i < VPT; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float xhat = (xv.v[i][e] - mu) * rstd;
          const float dyg = dyv.v[i][e] * g.v[i][e];
          xv.v[i][e] = xhat;
          s[0] += dyg;
          s[1] += dyg * xhat;
        }
      row_allreduce_sum<TPR, WG, 2>(s, slots, phase);
      c1 = s[0] * inv_n;
      c2 = s[1] * inv_n;
    } else {
      // One reduction per row instead of two: with d = x - shift (the shift is the row's
      // first element, see row_stats) the four sums of d, d^2, dy*gamma and dy*gamma*d give
      // the statistics and, through xhat = (d - mean_d) * rstd, both row sums of the gradient.
      const float shift = active ? sc0 : 0.f;
      float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const bool in_row = RowTile<T, VEC, TPR, VPT>::col(i, t) < cols;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float d = in_row ? xv.v[i][e] - shift : 0.f;
          const float dyg = dyv.v[i][e] * g.v[i][e];
          xv.v[i][e] = d;
          s[0] += d;
          s[1] += d * d;
          s[2] += dyg;
          s[3] += dyg * d;
        }
      }
      row_allreduce_sum<TPR, WG, 4>(s, slots, phase);
      const float md = s[0] * inv_n;
      const float var = fmaxf(s[1] * inv_n - md * md, 0.f);
      mu = shift + md;
      rstd = rsqrtf(var + eps);
      c1 = s[2] * inv_n;
      c2 = rstd * (s[3] - md * s[2]) * inv_n;
#pragma unroll
      for (int i = 0; i < VPT; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) xv.v[i][e] = (xv.v[i][e] - md) * rstd;  // xhat
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = RowTile<T, VEC, TPR, VPT>::col(i, t);
      float out[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float xhat = xv.v[i][e];
        const float d = dyv.v[i][e];
        out[e] = rstd * (d * g.v[i][e] - c1 - xhat * c2);
        acc_g.v[i][e] += d * xhat;
        acc_b.v[i][e] += d;
      }
      if (c < cols && active) {
        if (residual != nullptr) {
          // dx = round(gradient) + residual: bit for bit what a separate add of the stored
          // gradient gives.  `residual` may be `dx` itself (each element is read, then written,
          // by the same thread).
          float rs[VEC];
          VecIO<T, VEC>::load(residual + row * cols + c, rs);
          {
            // a plain addition, as the separate add kernel performs it: not to be contracted
            // with the multiplication that produced the gradient
#pragma clang fp contract(off)
#pragma unroll
            for (int e = 0; e < VEC; ++e) out[e] = to_float(from_float<T>(out[e])) + rs[e];
          }
        }
        VecIO<T, VEC>::store_stream(dx + row * cols + c, out);
      }
    }
    if constexpr (PREFETCH) {
      if (next < r_end) {
        xv = xn;
        dyv = dyn;
        sc0 = sc0_n;
        sc1 = sc1_n;
      }
    }
  }

  float* out_g = part_g + static_cast<int64_t>(blockIdx.x) * cols;
  float* out_b = part_b + static_cast<int64_t>(blockIdx.x) * cols;
  if constexpr (RPW == 1) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = RowTile<T, VEC, TPR, VPT>::col(i, t);
      if (c < cols) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          out_g[c + e] = acc_g.v[i][e];
          out_b[c + e] = acc_b.v[i][e];
        }
      }
    }
  } else {
    // The RPW row slots hold sums for the same columns: add them through LDS, dgamma first,
    // then dbeta through the same buffer.  Rows of 16 lanes: the four rows of a wave are
    // added inside the wave first (lanes l, l ^ 16, l ^ 32, l ^ 48 hold the same columns).
    if constexpr (TPR < kWave) {
#pragma unroll
      for (int i = 0; i < VPT; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
#pragma unroll
          for (int w = TPR; w < kWave; w *= 2) {
            acc_g.v[i][e] += __shfl_xor(acc_g.v[i][e], w);
            acc_b.v[i][e] += __shfl_xor(acc_b.v[i][e], w);
          }
        }
    }
    const int set = TPR < kWave ? static_cast<int>(threadIdx.x / kWave) : sub;
    const bool writer = TPR >= kWave || threadIdx.x % kWave < TPR;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
      const RowTile<T, VEC, TPR, VPT>& acc = which == 0 ? acc_g : acc_b;
      float* out = which == 0 ? out_g : out_b;
      if (which == 1) __syncthreads();
      if (writer) {
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
          const int c = (i * TPR + t) * VEC;
#pragma unroll
          for (int e = 0; e < VEC; ++e) combine[set * TILE_COLS + c + e] = acc.v[i][e];
        }
      }
      __syncthreads();
      for (int c = threadIdx.x; c < TILE_COLS && c < cols; c += WG) {
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < SETS; ++r) sum += combine[r * TILE_COLS + c];
        __builtin_nontemporal_store(sum, out + c);
      }
    }
  }
}

// ------------------------------------------------------------------------------------
// Fallback for rows too wide (or too oddly aligned) to hold in registers: one workgroup
// per row, streaming passes over global memory.  Writes dx and the row statistics; the
// column sums are then formed by ln_bwd_cols_kernel.
// ------------------------------------------------------------------------------------

template <typename T, int WG, bool HAS_STATS>
__global__ __launch_bounds__(WG) void ln_bwd_stream_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                           const T* __restrict__ gamma, const float* __restrict__ mean_in,
                                                           const float* __restrict__ rstd_in, T* __restrict__ dx,
                                                           float* __restrict__ mean_out, float* __restrict__ rstd_out,
                                                           int64_t rows, int64_t cols, float eps) {
  __shared__ float slots[2 * 2 * (WG / kWave)];
  int phase = 0;
  const int64_t row = blockIdx.x;
  if (row >= rows) return;
  const T* xr = x + row * cols;
  const T* dyr = dy + row * cols;
  float mu, rstd;
  if constexpr (HAS_STATS) {
    mu = mean_in[row];
    rstd = rstd_in[row];
  } else {
    const float shift = to_float(xr[0]);
    float s[2] = {0.f, 0.f};
    for (int64_t c = threadIdx.x; c < cols; c += WG) {
      const float d = to_float(xr[c]) - shift;
      s[0] += d;
      s[1] += d * d;
    }
    block_allreduce<SumOp, WG / kWave, 2>(s, slots, phase);
    phase ^= 1;
    const float inv_n = 1.0f / static_cast<float>(cols);
    const float md = s[0] * inv_n;
    mu = shift + md;
    rstd = rsqrtf(fmaxf(s[1] * inv_n - md * md, 0.f) + eps);
  }
  if (threadIdx.x == 0) {
    mean_out[row] = mu;
    rstd_out[row] = rstd;
  }
  float s[2] = {0.f, 0.f};
  for (int64_t c = threadIdx.x; c < cols; c += WG) {
    const float xhat = (to_float(xr[c]) - mu) * rstd;
    const float dyg = to_float(dyr[c]) * to_float(gamma[c]);
    s[0] += dyg;
    s[1] += dyg * xhat;
  }
  block_allreduce<SumOp, WG / kWave, 2>(s, slots, phase);
  const float inv_n = 1.0f / static_cast<float>(cols);
  const float c1 = s[0] * inv_n, c2 = s[1] * inv_n;
  for (int64_t c = threadIdx.x; c < cols; c += WG) {
    const float xhat = (to_float(xr[c]) - mu) * rstd;
    dx[row * cols + c] = from_float<T>(rstd * (to_float(dyr[c]) * to_float(gamma[c]) - c1 - xhat * c2));
  }
}

// Partial column sums of dy*xhat and dy over a slab of rows; thread = one column.
template <typename T, int WG>
__global__ __launch_bounds__(WG) void ln_bwd_cols_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                         const float* __restrict__ mean, const float* __restrict__ rstd,
                                                         float* __restrict__ part_g, float* __restrict__ part_b,
                                                         int64_t rows, int64_t cols, int64_t rows_per_group) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * WG + threadIdx.x;
  if (c >= cols) return;
  const int64_t r_begin = static_cast<int64_t>(blockIdx.y) * rows_per_group;
  const int64_t r_end = min(r_begin + rows_per_group, rows);
  float sg = 0.f, sb = 0.f;
  for (int64_t r = r_begin; r < r_end; ++r) {
    const float d = to_float(dy[r * cols + c]);
    sg += d * (to_float(x[r * cols + c]) - mean[r]) * rstd[r];
    sb += d;
  }
  part_g[static_cast<int64_t>(blockIdx.y) * cols + c] = sg;
  part_b[static_cast<int64_t>(blockIdx.y) * cols + c] = sb;
}

// ------------------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------------------

template <typename T>
struct LayerNormOps {
  static constexpr int WIDE = WideVec<T>::value;

  // How a row of `chunks` chunks is laid over threads.
  struct Shape {
    int tpr, vpt;
  };
  // The backward keeps one wave per row from 33 chunks on: with three chunks per lane its five
  // row tiles no longer fit a 1024-thread workgroup, and sixteen-lane rows in smaller
  // workgroups measured slower there ((16384, 384) bf16, row kernel alone: 16.7 us with 256
  // threads and 20.4 us with 512 against 13.8 us).
  static bool pick_shape_bwd(int64_t chunks, Shape* s) {
    if (chunks > 32 && chunks <= 64) {
      *s = {64, 1};
      return true;
    }
    return pick_shape(chunks, s);
  }
  static bool pick_shape(int64_t chunks, Shape* s) {
    // Up to 48 chunks: sixteen lanes per row, four rows per wave (a 384-column 16-bit row is
    // 48 chunks: one wave per row would leave a quarter of the lanes idle and need the
    // cross-row steps of the wave reduction).
    if (chunks <= 16) *s = {16, 1};
    else if (chunks <= 32) *s = {16, 2};
    else if (chunks <= 48) *s = {16, 3};
    else if (chunks <= 64) *s = {64, 1};
    else if (chunks <= 128) *s = {64, 2};
    else if (chunks <= 256) *s = {64, 4};
    else if (chunks <= 512) *s = {256, 2};
    else if (chunks <= 1024) *s = {512, 2};
    else if (chunks <= 2048) *s = {512, 4};
    else if (chunks <= 4096) *s = {1024, 4};
    else if (chunks <= 8192) *s = {1024, 8};
    else return false;
    return true;
  }

  static bool can_vectorise(int64_t cols, std::initializer_list<const void*> ptrs) {
    if (WIDE == 1 || cols % WIDE != 0) return false;
    for (const void* p : ptrs)
      if (p != nullptr && !aligned16(p)) return false;
    return true;
  }

  template <int VEC, int TPR, int VPT>
  static int launch_fwd(const T* x, const T* gamma, const T* beta, T* y, float* mean, float* rstd, int64_t rows,
                        int64_t cols, float eps, hipStream_t stream) {
    constexpr int WG = TPR <= 64 ? 256 : TPR;
    constexpr int RPW = WG / TPR;
    const int64_t want = ceil_div(rows, RPW);
    const int64_t cap = static_cast<int64_t>(device_info().cu_count) * env_int("MOGRAD_HIP_LN_FWD_WG_PER_CU", 4);
    const unsigned grid = static_cast<unsigned>(want < cap ? want : cap);
    hipLaunchKernelGGL((ln_fwd_rows_kernel<T, VEC, TPR, VPT, WG>), dim3(grid), dim3(WG), 0, stream, x, gamma, beta, y,
                       mean, rstd, rows, static_cast<int>(cols), eps);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }

  template <int VEC>
  static int dispatch_fwd(Shape s, const T* x, const T* gamma, const T* beta, T* y, float* mean, float* rstd,
                          int64_t rows, int64_t cols, float eps, hipStream_t stream) {
#define MG_LN_FWD_CASE(TPR_, VPT_) \
  if (s.tpr == TPR_ && s.vpt == VPT_) return launch_fwd<VEC, TPR_, VPT_>(x, gamma, beta, y, mean, rstd, rows, cols, eps, stream)
    MG_LN_FWD_CASE(16, 1);
    MG_LN_FWD_CASE(16, 2);
    MG_LN_FWD_CASE(16, 3);
    MG_LN_FWD_CASE(64, 1);
    MG_LN_FWD_CASE(64, 2);
    MG_LN_FWD_CASE(64, 4);
    MG_LN_FWD_CASE(256, 2);
    MG_LN_FWD_CASE(512, 2);
    MG_LN_FWD_CASE(512, 4);
    MG_LN_FWD_CASE(1024, 4);
    MG_LN_FWD_CASE(1024, 8);
#undef MG_LN_FWD_CASE
    return fail(MG_ERR_UNSUPPORTED, "layer_norm_fwd: no kernel for row shape (%d, %d)", s.tpr, s.vpt);
  }

  static int fwd(const void* x_, const void* gamma_, const void* beta_, void* y_, float* mean, float* rstd,
                 int64_t rows, int64_t cols, float eps, hipStream_t stream) {
    const T* x = static_cast<const T*>(x_);
    const T* gamma = static_cast<const T*>(gamma_);
    const T* beta = static_cast<const T*>(beta_);
    T* y = static_cast<T*>(y_);
    Shape s;
    if (can_vectorise(cols, {x, gamma, beta, y}) && pick_shape(cols / WIDE, &s))
      return dispatch_fwd<WIDE>(s, x, gamma, beta, y, mean, rstd, rows, cols, eps, stream);
    if (pick_shape(cols, &s)) return dispatch_fwd<1>(s, x, gamma, beta, y, mean, rstd, rows, cols, eps, stream);
    hipLaunchKernelGGL((ln_fwd_stream_kernel<T, 1024>), dim3(static_cast<unsigned>(rows)), dim3(1024), 0, stream, x,
                       gamma, beta, y, mean, rstd, rows, cols, eps);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }

  // Number of row groups for the backward: enough workgroups to fill the device, few
  // enough that the (groups, cols) partial sums stay a small fraction of the traffic.
  static int64_t bwd_groups(int64_t rows, int rows_per_iter, int wg) {
    const int64_t cus = device_info().cu_count;
    int64_t per_cu = wg >= 1024 ? 1 : (wg >= 256 ? 2 : 4);
    per_cu = env_int("MOGRAD_HIP_LN_GROUPS_PER_CU", static_cast<int>(per_cu));
    int64_t groups = cus * per_cu;
    const int64_t max_groups = ceil_div(rows, rows_per_iter);
    if (groups > max_groups) groups = max_groups;
    if (groups < 1) groups = 1;
    return groups;
  }

  // WG: threads per workgroup; TPR of them share a row, so WG / TPR rows are in flight per
  // workgroup.  One-wave rows (TPR = 64) of tall matrices use 1024 threads: sixteen rows in
  // flight per workgroup cover the load latency that four do not, and the number of partial
  // sums (one set per workgroup) stays the same.
  template <int VEC, int TPR, int VPT, bool HAS_STATS, int WG_ = 0>
  static int launch_bwd(const T* dy, const T* x, const T* gamma, const float* mean, const float* rstd,
                        const T* residual, T* dx, T* dgamma, T* dbeta, int64_t rows, int64_t cols, float eps,
                        hipStream_t stream) {
    if constexpr (TPR == 512 && VPT * VEC <= 8 && WG_ == 0) {
      // Rows of 512 threads in pairs, one 1024-thread workgroup per CU instead of two of 512:
      // as many rows in flight, half as many partial dgamma/dbeta sums to write and read back
      // ((2048, 4096) fp32: 25.2 -> 23.5 us on cached inputs, 1-4 % on cold ones; (1024, 4096):
      // 18.8 -> 15.8 us).  Only for tiles of
      // up to 8 values per thread: wider ones do not fit the registers of a 1024-thread
      // workgroup (16 values: 2 % slower, 32 values: spills, 4x slower).
      // MOGRAD_HIP_LN_WIDE_PAIR=0 keeps single rows.
      if (rows >= 4 * static_cast<int64_t>(device_info().cu_count) && env_int("MOGRAD_HIP_LN_WIDE_PAIR", 1) != 0)
        return launch_bwd<VEC, TPR, VPT, HAS_STATS, 1024>(dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta, rows,
                                                          cols, eps, stream);
    }
    if constexpr (TPR <= 64 && WG_ == 0) {
      // The largest workgroup whose register budget holds the five row tiles: 1024 threads
      // (128 registers) up to 8 values per tile, 512 up to 16, 256 beyond.
      constexpr int TALL_WG = VPT * VEC <= 8 ? 1024 : (VPT * VEC <= 16 ? 512 : 256);
      const int64_t tall = static_cast<int64_t>(device_info().cu_count) * env_int("MOGRAD_HIP_LN_TALL_ROWS_PER_CU", 16);
      if (rows >= tall && TALL_WG > 256)
        return launch_bwd<VEC, TPR, VPT, HAS_STATS, TALL_WG>(dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta,
                                                             rows, cols, eps, stream);
    }
    constexpr int WG = WG_ != 0 ? WG_ : (TPR <= 64 ? 256 : TPR);
    constexpr int RPW = WG / TPR;
    int64_t groups = bwd_groups(rows, RPW, WG);
    int64_t rows_per_group = ceil_div(ceil_div(rows, groups), RPW) * RPW;
    groups = ceil_div(rows, rows_per_group);
    // Matrices of 16 MiB and more: the groups' rows interleaved, so that the workgroups of one
    // trip read a contiguous band of x and dy and write one of dx (DRAM pages shared between
    // neighbours: (16384, 1024) fp32 47.4 -> 43.6 us, (4096, 8192) bf16 62.8 -> 59.3 us,
    // (2048, 4096) fp32 29.6 -> 28.5 us).  Smaller, cache-resident ones measure 1 % slower that
    // way and keep consecutive rows.  MOGRAD_HIP_LN_INTERLEAVE=0/1 forces either.
    const int il_knob = env_int("MOGRAD_HIP_LN_INTERLEAVE", -1);
    const bool interleave =
        il_knob < 0 ? rows * cols * static_cast<int64_t>(sizeof(T)) >= (int64_t{16} << 20) : il_knob != 0;
    Scratch part_g, part_b;
    MG_TRY(part_g.take(groups * cols * static_cast<int64_t>(sizeof(float))));
    MG_TRY(part_b.take(groups * cols * static_cast<int64_t>(sizeof(float))));
    hipLaunchKernelGGL((ln_bwd_rows_kernel<T, VEC, TPR, VPT, WG, HAS_STATS>), dim3(static_cast<unsigned>(groups)),
                       dim3(WG), 0, stream, dy, x, gamma, mean, rstd, residual, dx, part_g.as<float>(),
                       part_b.as<float>(), rows,
                       static_cast<int>(cols), eps, rows_per_group,
                       interleave ? groups * RPW : static_cast<int64_t>(RPW));
    MG_LAUNCH_CHECK();
    reduce_partials_or_defer<T>(part_g, dgamma, &part_b, dbeta, groups, cols, device_info().cu_count, stream);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }

  template <int VEC, bool HAS_STATS>
  static int dispatch_bwd(Shape s, const T* dy, const T* x, const T* gamma, const float* mean, const float* rstd,
                          const T* residual, T* dx, T* dgamma, T* dbeta, int64_t rows, int64_t cols, float eps,
                          hipStream_t stream) {
#define MG_LN_BWD_CASE(TPR_, VPT_)       \
  if (s.tpr == TPR_ && s.vpt == VPT_)    \
  return launch_bwd<VEC, TPR_, VPT_, HAS_STATS>(dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta, rows, cols, eps, \
                                                stream)
    MG_LN_BWD_CASE(16, 1);
    MG_LN_BWD_CASE(16, 2);
    MG_LN_BWD_CASE(64, 1);
    MG_LN_BWD_CASE(64, 2);
    MG_LN_BWD_CASE(64, 4);
    MG_LN_BWD_CASE(256, 2);
    MG_LN_BWD_CASE(512, 2);
    MG_LN_BWD_CASE(512, 4);
    MG_LN_BWD_CASE(1024, 4);
#undef MG_LN_BWD_CASE
    return fail(MG_ERR_UNSUPPORTED, "layer_norm_bwd: no kernel for row shape (%d, %d)", s.tpr, s.vpt);
  }

  template <bool HAS_STATS>
  static int bwd_stream(const T* dy, const T* x, const T* gamma, const float* mean, const float* rstd, T* dx,
                        T* dgamma, T* dbeta, int64_t rows, int64_t cols, float eps, hipStream_t stream) {
    constexpr int WG = 1024;
    Scratch stat_mean, stat_rstd, part_g, part_b;
    MG_TRY(stat_mean.take(rows * static_cast<int64_t>(sizeof(float))));
    MG_TRY(stat_rstd.take(rows * static_cast<int64_t>(sizeof(float))));
    hipLaunchKernelGGL((ln_bwd_stream_kernel<T, WG, HAS_STATS>), dim3(static_cast<unsigned>(rows)), dim3(WG), 0, stream,
                       dy, x, gamma, mean, rstd, dx, stat_mean.as<float>(), stat_rstd.as<float>(), rows, cols, eps);
    MG_LAUNCH_CHECK();
    const int64_t col_blocks = ceil_div(cols, 256);
    int64_t groups = ceil_div(static_cast<int64_t>(device_info().cu_count) * 4, col_blocks);
    if (groups > rows) groups = rows;
    if (groups < 1) groups = 1;
    const int64_t rows_per_group = ceil_div(rows, groups);
    groups = ceil_div(rows, rows_per_group);
    MG_TRY(part_g.take(groups * cols * static_cast<int64_t>(sizeof(float))));
    MG_TRY(part_b.take(groups * cols * static_cast<int64_t>(sizeof(float))));
    hipLaunchKernelGGL((ln_bwd_cols_kernel<T, 256>), dim3(static_cast<unsigned>(col_blocks), static_cast<unsigned>(groups)),
                       dim3(256), 0, stream, dy, x, stat_mean.as<float>(), stat_rstd.as<float>(), part_g.as<float>(),
                       part_b.as<float>(), rows, cols, rows_per_group);
    MG_LAUNCH_CHECK();
    reduce_partials_or_defer<T>(part_g, dgamma, &part_b, dbeta, groups, cols, device_info().cu_count, stream);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }

  // `residual` (optional, may alias dx): dx = round(gradient) + residual.
  template <bool HAS_STATS>
  static int bwd(const void* dy_, const void* x_, const void* gamma_, const float* mean, const float* rstd,
                 const void* residual_, void* dx_, void* dgamma_, void* dbeta_, int64_t rows, int64_t cols, float eps,
                 int dtype, hipStream_t stream) {
    const T* residual = static_cast<const T*>(residual_);
    const T* dy = static_cast<const T*>(dy_);
    const T* x = static_cast<const T*>(x_);
    const T* gamma = static_cast<const T*>(gamma_);
    T* dx = static_cast<T*>(dx_);
    T* dgamma = static_cast<T*>(dgamma_);
    T* dbeta = static_cast<T*>(dbeta_);
    Shape s;
    // The backward keeps five row tiles per thread: at most 16 elements per tile with
    // 1024 threads (128 registers each), 32 with fewer threads.  Wider rows stream.
    auto fits = [](const Shape& sh, int vec) { return sh.vpt * vec <= (sh.tpr == 1024 ? 16 : 32); };
    if (can_vectorise(cols, {dy, x, gamma, dx, residual}) && pick_shape_bwd(cols / WIDE, &s) && fits(s, WIDE))
      return dispatch_bwd<WIDE, HAS_STATS>(s, dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta, rows, cols, eps,
                                           stream);
    if (pick_shape_bwd(cols, &s) && fits(s, 1))
      return dispatch_bwd<1, HAS_STATS>(s, dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta, rows, cols, eps, stream);
    if (residual == nullptr)
      return bwd_stream<HAS_STATS>(dy, x, gamma, mean, rstd, dx, dgamma, dbeta, rows, cols, eps, stream);
    // Streaming fallback: the gradient goes to scratch first (the residual may be dx itself), then one add.
    Scratch tmp;
    MG_TRY(tmp.take(rows * cols * static_cast<int64_t>(sizeof(T))));
    MG_TRY(bwd_stream<HAS_STATS>(dy, x, gamma, mean, rstd, tmp.as<T>(), dgamma, dbeta, rows, cols, eps, stream));
    return mg_add(tmp.as<T>(), residual, dx, rows * cols, dtype, stream);
  }
};

}  // namespace mg

// Defines the per-dtype entry points that layer_norm.hip dispatches to.
#define MG_DEFINE_LAYER_NORM(T, SUFFIX)                                                                          \
  namespace mg {                                                                                                 \
  int ln_fwd_##SUFFIX(const void* x, const void* gamma, const void* beta, void* y, float* mean, float* rstd,     \
                      int64_t rows, int64_t cols, float eps, hipStream_t stream) {                               \
    return LayerNormOps<T>::fwd(x, gamma, beta, y, mean, rstd, rows, cols, eps, stream);                         \
  }                                                                                                              \
  int ln_bwd_##SUFFIX(const void* dy, const void* x, const void* gamma, const float* mean, const float* rstd,    \
                      const void* residual, void* dx, void* dgamma, void* dbeta, int64_t rows, int64_t cols,     \
                      float eps, int dtype, hipStream_t stream) {                                                \
    if (mean != nullptr)                                                                                         \
      return LayerNormOps<T>::template bwd<true>(dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta, rows,    \
                                                 cols, eps, dtype, stream);                                      \
    return LayerNormOps<T>::template bwd<false>(dy, x, gamma, mean, rstd, residual, dx, dgamma, dbeta, rows,     \
                                                cols, eps, dtype, stream);                                       \
  }                                                                                                              \
  }
