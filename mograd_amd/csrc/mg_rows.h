// Building blocks shared by the row-oriented kernels (LayerNorm, cross-entropy, column
// sums): a register-resident row tile, the reduction over the threads sharing a row, and
// the second stage of the two-stage column reduction.
#pragma once

#include "mg_deferred.h"
#include "mg_device.h"

namespace mg {

// ------------------------------------------------------------------------------------
// Row tile: VPT chunks of VEC elements per thread.
// ------------------------------------------------------------------------------------

template <typename T, int VEC, int TPR, int VPT>
struct RowTile {
  float v[VPT][VEC];

  // Column of element 0 of this thread's chunk i.  Rows are narrower than 2^31 elements
  // (checked on the host), so 32-bit column arithmetic is enough.
  static __device__ __forceinline__ int col(int i, int t) { return (i * TPR + t) * VEC; }

  // Number of leading chunk indices i for which every one of the TPR threads has a valid
  // chunk.  It is wave-uniform, so "i < full_chunks(cols)" is a scalar branch: only chunk
  // index full_chunks(cols) needs per-lane predication, later ones are absent.
  static __device__ __forceinline__ int full_chunks(int cols) { return (cols / VEC) / TPR; }

  // Addresses are formed as (uniform row pointer + chunk offset) + (unsigned lane offset),
  // the shape the compiler can turn into scalar-base + 32-bit-vector-offset memory
  // instructions, so that no per-chunk 64-bit address registers are kept.
  __device__ __forceinline__ void load(const T* row_ptr, int t, int cols) {
    const unsigned lane_off = static_cast<unsigned>(t) * VEC;
    const int nfull = full_chunks(cols);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const T* chunk_base = row_ptr + i * (TPR * VEC);
      if (i < nfull) {
        VecIO<T, VEC>::load(chunk_base + lane_off, v[i]);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[i][e] = 0.f;
        if (i == nfull && col(i, t) < cols) VecIO<T, VEC>::load(chunk_base + lane_off, v[i]);
      }
    }
  }
  __device__ __forceinline__ void store(T* row_ptr, int t, int cols) const {
    const unsigned lane_off = static_cast<unsigned>(t) * VEC;
    const int nfull = full_chunks(cols);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      T* chunk_base = row_ptr + i * (TPR * VEC);
      if (i < nfull) {
        VecIO<T, VEC>::store(chunk_base + lane_off, v[i]);
      } else if (i == nfull && col(i, t) < cols) {
        VecIO<T, VEC>::store(chunk_base + lane_off, v[i]);
      }
    }
  }
  // The same with stores that bypass the caches (see VecIO::store_stream).
  __device__ __forceinline__ void store_stream(T* row_ptr, int t, int cols) const {
    const unsigned lane_off = static_cast<unsigned>(t) * VEC;
    const int nfull = full_chunks(cols);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      T* chunk_base = row_ptr + i * (TPR * VEC);
      if (i < nfull) {
        VecIO<T, VEC>::store_stream(chunk_base + lane_off, v[i]);
      } else if (i == nfull && col(i, t) < cols) {
        VecIO<T, VEC>::store_stream(chunk_base + lane_off, v[i]);
      }
    }
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < VPT; ++i)
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[i][e] = 0.f;
  }
};

// Reduction over the TPR threads that share a row: wave-only when TPR == 64, the whole
// workgroup when TPR == WG, otherwise TPR / 64 consecutive waves of it.
// Position of a thread among the TPR threads of its row, and which of the WG/TPR row
// slots of the workgroup it serves.  With one row per workgroup the slot is the constant
// 0, which keeps row addresses wave-uniform (scalar registers).
template <int TPR, int WG>
__device__ __forceinline__ void row_thread(int& t, int& sub) {
  if constexpr (TPR == WG) {
    t = threadIdx.x;
    sub = 0;
  } else {
    t = threadIdx.x % TPR;
    sub = threadIdx.x / TPR;
  }
}

template <int TPR, int WG, int K>
__device__ __forceinline__ void row_allreduce_sum(float (&v)[K], float* slots, int& phase) {
  if constexpr (TPR == 16) {
    // four rows side by side in a wave, each on one row of 16 lanes
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = row16_allreduce<SumOp>(v[k]);
  } else if constexpr (TPR == kWave) {
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = wave_sum(v[k]);
  } else if constexpr (TPR == WG) {
    block_allreduce<SumOp, WG / kWave, K>(v, slots, phase);
    phase ^= 1;
  } else {
    group_allreduce<SumOp, WG / kWave, TPR / kWave, K>(v, slots, phase);
    phase ^= 1;
  }
}

// ------------------------------------------------------------------------------------
// Second stage of a column reduction: out[c] = sum_g part[g][c], plain stores, fixed
// order (used by LayerNorm's dgamma/dbeta and by the bias gradient).
// Workgroup = CW columns x 256/CW row slices; blockIdx.y selects which of up to two
// (partials, output) pairs to reduce.
// ------------------------------------------------------------------------------------

// One workgroup's share (256 threads, `tid` of them; column block `bx`) of the sum below.
// `tile` is SL x CW floats of LDS.  Every thread of the 256 must make the call: it holds
// barriers.
template <typename T, int CW>
__device__ __forceinline__ void reduce_partials_cw_block(float* __restrict__ tile_, int tid, int64_t bx,
                                                         const float* __restrict__ part, T* __restrict__ out,
                                                         int64_t groups, int64_t cols) {
  constexpr int SL = 256 / CW;  // row slices per workgroup
  float(&tile)[SL][CW] = *reinterpret_cast<float(*)[SL][CW]>(tile_);
  const int cx = tid % CW;
  const int sy = tid / CW;
  const int64_t c = bx * CW + cx;
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  if (c < cols) {
    int64_t g = sy;
    for (; g + 3 * SL < groups; g += 4 * SL) {
      a0 += part[g * cols + c];
      a1 += part[(g + SL) * cols + c];
      a2 += part[(g + 2 * SL) * cols + c];
      a3 += part[(g + 3 * SL) * cols + c];
    }
    for (; g < groups; g += SL) a0 += part[g * cols + c];
  }
  tile[sy][cx] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  // fixed-order tree over the slices
#pragma unroll
  for (int w = SL / 2; w > 0; w /= 2) {
    if (sy < w) tile[sy][cx] += tile[sy + w][cx];
    __syncthreads();
  }
  if (sy == 0 && c < cols) out[c] = from_float<T>(tile[0][cx]);
}

template <typename T, int CW>
__global__ __launch_bounds__(256) void reduce_partials_cw_kernel(const float* __restrict__ part0, T* __restrict__ out0,
                                                                 const float* __restrict__ part1, T* __restrict__ out1,
                                                                 int64_t groups, int64_t cols) {
  __shared__ float tile[256];
  reduce_partials_cw_block<T, CW>(tile, threadIdx.x, blockIdx.x, blockIdx.y == 0 ? part0 : part1,
                                  blockIdx.y == 0 ? out0 : out1, groups, cols);
}

// The same sum for wide outputs with many groups: a 1024-thread workgroup owns 32 columns
// (one 128-byte line of the fp32 partials) and reads them as 16-byte pieces, eight pieces
// by 128 group lanes, so that a few hundred groups are in flight at once instead of being
// walked four at a time; the group lanes are then added through LDS in a fixed order.
// Needs cols % 4 == 0 and 16-byte aligned partials.
constexpr int kSlabLanes = 128, kSlabCols = 32, kSlabSlices = 32;
constexpr int kSlabLdsFloats = (kSlabLanes + kSlabSlices) * (kSlabCols + 1);
// One 1024-thread workgroup's share (column block `bx`); `lds` is kSlabLdsFloats floats.
template <typename T>
__device__ __forceinline__ void reduce_partials_slab_block(float* __restrict__ lds, int64_t bx,
                                                           const float* __restrict__ part, T* __restrict__ out,
                                                           int64_t groups, int64_t cols) {
  constexpr int LANES = kSlabLanes, NCOL = kSlabCols, SL = kSlabSlices;
  float(&tile)[LANES][NCOL + 1] = *reinterpret_cast<float(*)[LANES][NCOL + 1]>(lds);
  float(&tile2)[SL][NCOL + 1] = *reinterpret_cast<float(*)[SL][NCOL + 1]>(lds + LANES * (NCOL + 1));
  const int cx = threadIdx.x % 8;
  const int ly = threadIdx.x / 8;
  const int64_t col = (bx * 8 + cx) * 4;
  float4 a0 = make_float4(0.f, 0.f, 0.f, 0.f), a1 = a0;
  if (col < cols) {
    const float* p = part + ly * cols + col;
    const int64_t step = LANES * cols;
    int64_t g = ly;
    for (; g + LANES < groups; g += 2 * LANES, p += 2 * step) {
      const mg_f4 v0 = __builtin_nontemporal_load(reinterpret_cast<const mg_f4*>(p));
      const mg_f4 v1 = __builtin_nontemporal_load(reinterpret_cast<const mg_f4*>(p + step));
      a0.x += v0.x; a0.y += v0.y; a0.z += v0.z; a0.w += v0.w;
      a1.x += v1.x; a1.y += v1.y; a1.z += v1.z; a1.w += v1.w;
    }
    if (g < groups) {
      const mg_f4 v0 = __builtin_nontemporal_load(reinterpret_cast<const mg_f4*>(p));
      a0.x += v0.x; a0.y += v0.y; a0.z += v0.z; a0.w += v0.w;
    }
  }
  tile[ly][cx * 4 + 0] = a0.x + a1.x;
  tile[ly][cx * 4 + 1] = a0.y + a1.y;
  tile[ly][cx * 4 + 2] = a0.z + a1.z;
  tile[ly][cx * 4 + 3] = a0.w + a1.w;
  __syncthreads();
  {
    const int c = threadIdx.x % NCOL, sl = threadIdx.x / NCOL;
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < LANES / SL; ++k) t += tile[sl * (LANES / SL) + k][c];
    tile2[sl][c] = t;
  }
  __syncthreads();
  if (threadIdx.x < NCOL) {
    const int64_t c = bx * NCOL + threadIdx.x;
    float t = 0.f;
#pragma unroll
    for (int sl = 0; sl < SL; ++sl) t += tile2[sl][threadIdx.x];
    if (c < cols) out[c] = from_float<T>(t);
  }
}

template <typename T>
__global__ __launch_bounds__(1024) void reduce_partials_slab_kernel(const float* __restrict__ part0, T* __restrict__ out0,
                                                                    const float* __restrict__ part1, T* __restrict__ out1,
                                                                    int64_t groups, int64_t cols) {
  __shared__ float lds[kSlabLdsFloats];
  reduce_partials_slab_block<T>(lds, blockIdx.x, blockIdx.y == 0 ? part0 : part1, blockIdx.y == 0 ? out0 : out1, groups,
                                cols);
}

// Launches the reduction of one or two (groups, cols) partial arrays.  With at least 128
// groups of 16-byte aligned rows the slab kernel takes it (every partial in flight at once:
// about 1 us less per call than the forms below at 256 groups, for 384 columns as for
// 4096).  Otherwise wide outputs use 64
// columns x 4 slices per workgroup; narrower ones 32 x 8 (a workgroup still reads whole
// 128-byte lines of the fp32 partials: with 64-byte pieces the two workgroups that share a
// line sit on different XCDs and each L2 fetches the line, which doubled the kernel's
// fetched bytes at 4096 columns); a few hundred columns use 16 x 16 so that they still
// spread over enough workgroups to hide the load latency.
// Which form sums (groups, cols) partials: 0 the slab kernel, else the column width of
// reduce_partials_cw_kernel.
inline int reduce_partials_variant(const float* part0, const float* part1, int64_t groups, int64_t cols, int cu_count) {
  const int64_t pairs = part1 ? 2 : 1;
  const bool slab_ok = cols % 4 == 0 && groups >= 128 && aligned16(part0) && (!part1 || aligned16(part1)) &&
                       env_int("MOGRAD_HIP_REDUCE_SLAB", 1) != 0;
  if (slab_ok) return 0;
  if (ceil_div(cols, 64) * pairs >= static_cast<int64_t>(cu_count)) return 64;
  if (ceil_div(cols, 32) * pairs * 2 >= static_cast<int64_t>(cu_count)) return 32;
  return 16;
}

template <typename T>
inline void launch_reduce_partials(const float* part0, T* out0, const float* part1, T* out1, int64_t groups, int64_t cols,
                                   int cu_count, hipStream_t stream) {
  const unsigned pairs = part1 ? 2u : 1u;
  const int variant = reduce_partials_variant(part0, part1, groups, cols, cu_count);
  if (variant == 0) {
    hipLaunchKernelGGL((reduce_partials_slab_kernel<T>), dim3(static_cast<unsigned>(ceil_div(cols, 32)), pairs),
                       dim3(1024), 0, stream, part0, out0, part1, out1, groups, cols);
  } else if (variant == 64) {
    hipLaunchKernelGGL((reduce_partials_cw_kernel<T, 64>), dim3(static_cast<unsigned>(ceil_div(cols, 64)), pairs),
                       dim3(256), 0, stream, part0, out0, part1, out1, groups, cols);
  } else if (variant == 32) {
    hipLaunchKernelGGL((reduce_partials_cw_kernel<T, 32>), dim3(static_cast<unsigned>(ceil_div(cols, 32)), pairs),
                       dim3(256), 0, stream, part0, out0, part1, out1, groups, cols);
  } else {
    hipLaunchKernelGGL((reduce_partials_cw_kernel<T, 16>), dim3(static_cast<unsigned>(ceil_div(cols, 16)), pairs),
                       dim3(256), 0, stream, part0, out0, part1, out1, groups, cols);
  }
}

// launch_reduce_partials, unless a `_deferred` entry point is running on this thread: then the
// sums are recorded on its list (same form, hence the same order of additions) together with
// the partials' pool blocks, and nothing is launched here.
template <typename T>
inline void reduce_partials_or_defer(Scratch& part0, T* out0, Scratch* part1, T* out1, int64_t groups, int64_t cols,
                                     int cu_count, hipStream_t stream) {
  const float* p0 = part0.as<float>();
  const float* p1 = part1 ? part1->as<float>() : nullptr;
  DeferredList* dl = deferred_current();
  if (!dl || cols > 0x7fffffffLL || groups > 0x7fffffffLL) {
    launch_reduce_partials<T>(p0, out0, p1, out1, groups, cols, cu_count, stream);
    return;
  }
  const int variant = reduce_partials_variant(p0, p1, groups, cols, cu_count);
  const int kind = variant == 0 ? kDeferSlab : variant == 64 ? kDeferCw64 : variant == 32 ? kDeferCw32 : kDeferCw16;
  const int64_t blocks = deferred_column_blocks(variant, cols);
  dl->push(kind, p0, out0, 0, 0, static_cast<int>(cols), static_cast<int>(groups), blocks);
  if (p1) dl->push(kind, p1, out1, 0, 0, static_cast<int>(cols), static_cast<int>(groups), blocks);
  dl->hold(part0);
  if (part1) dl->hold(*part1);
}

}  // namespace mg
