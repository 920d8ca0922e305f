// Matrix products C = A x B (+ bias) for the Linear forward and its gradients.
//
// An operand is described by which of its two dimensions is contiguous in memory:
//   A (M x K): "k-contiguous"  A[m * lda + k]   (a row-major (M,K) array), or
//              "m-contiguous"  A[k * lda + m]   (the transposed view of a (K,M) array)
//   B (K x N): "k-contiguous"  B[n * ldb + k]   (a row-major (N,K) array, i.e. B^T given), or
//              "n-contiguous"  B[k * ldb + n]   (a row-major (K,N) array)
// so Y = X W^T is (k,k), dX = dY W is (k,n) and dW = dY^T X is (m,n), all without
// materialising a transpose.  C is row-major (M,N) with leading dimension ldc.
//
// fp32 kernel: 128x128 output tile per 256-thread workgroup, four waves in a 2x2 grid,
// each wave a 64x64 tile as 2x2 v_mfma_f32_32x32x2_f32 accumulators (64 registers).
// A K-chunk of 32 is staged through LDS: global -> registers (prefetch of the next
// chunk overlaps the MFMAs of the current one) -> LDS -> MFMA operands.
#pragma once

#include <type_traits>

#include "mg_device.h"
#include "mg_internal.h"

namespace mg {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kGemmBM = 128;
constexpr int kGemmBN = 128;
constexpr int kGemmBK = 32;
constexpr int kGemmThreads = 256;
constexpr int kKcStride = kGemmBK + 4;  // floats per LDS row of a k-contiguous operand tile

// Workgroup -> output tile.  Consecutive workgroup ids go to different XCDs (id % 8), each
// with its own L2; ids are regrouped so that one XCD works on a compact block of tiles
// that share operand rows and columns.
constexpr int kXcd = 8;
__device__ __forceinline__ void gemm_tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn,
                                                   bool regroup = true) {
  const int total = tiles_m * tiles_n;
  int id = bid;
  if (regroup && total % kXcd == 0) id = (bid % kXcd) * (total / kXcd) + bid / kXcd;
  // Raster in bands of 4 tile-rows so that a band's A rows stay in L2.
  constexpr int kBand = 4;
  const int band_tiles = kBand * tiles_n;
  const int band = id / band_tiles;
  const int in_band = id % band_tiles;
  const int rows_here = min(kBand, tiles_m - band * kBand);
  tm = band * kBand + in_band % rows_here;
  tn = in_band / rows_here;
}

// Split-K launches use one grid axis.  The work items, one per (batch, K range, output tile),
// are numbered with the tile varying fastest, and XCD x (the workgroups whose id is x mod kXcd)
// takes the contiguous block [x n / kXcd, (x + 1) n / kXcd) of the n items: every XCD gets the
// same number of items to within one (dealing out whole K ranges left two XCDs with twice the
// work of the others whenever the ranges were no multiple of eight), and an XCD's items are
// mostly whole K ranges, whose tiles read the same rows of both operands, so a range is fetched
// into one or two L2s instead of all eight (the dW of a 384 -> 1536 layer over 16384 rows
// fetched 240 MB for 63 MB of operands with tiles dealt out round robin).  Returns false for
// the few padding workgroups at the end of the shorter blocks.
__device__ __forceinline__ bool gemm_split_work(int bid, int tiles, int splits, int batches, int& tile, int& split,
                                                int& batch) {
  const int64_t n = static_cast<int64_t>(tiles) * splits * batches;
  const int x = bid % kXcd;
  const int64_t item = x * n / kXcd + bid / kXcd;
  if (item >= (x + 1) * n / kXcd) return false;
  const int group = static_cast<int>(item / tiles);
  tile = static_cast<int>(item % tiles);
  split = group % splits;
  batch = group / splits;
  return true;
}
inline int64_t gemm_split_grid(int64_t tiles, int64_t splits, int64_t batches) {
  return kXcd * ((tiles * splits * batches + kXcd - 1) / kXcd);
}

// What happens to a product element after the bias: v = acc + bias; relu: v = max(v, 0);
// relu_mask (laid out like C): v = 0 where mask <= 0; v is rounded to T; residual (laid out
// like C, may be C itself): v = round(v + residual).  For 16-bit types the residual is added
// to the rounded product, which is bit for bit what a separate add kernel computes.
template <typename T>
struct GemmEpilogue {
  const T* residual;
  const T* relu_mask;
  int relu;
};

template <typename T>
__device__ __forceinline__ T gemm_finish(float v, const GemmEpilogue<T>& ep, int64_t index) {
  if (ep.relu) v = v > 0.f ? v : 0.f;
  if (ep.relu_mask) v = to_float(ep.relu_mask[index]) > 0.f ? v : 0.f;
  T out = from_float<T>(v);
  if (ep.residual) out = from_float<T>(to_float(out) + to_float(ep.residual[index]));
  return out;
}

// Registers holding one thread's share of a 128 x 32 (or 32 x 128) operand tile.
struct GemmStage {
  float4 v[4];
};

// Loads the tile of an operand whose "outer" index (m for A, n for B) starts at `o0` and
// whose k index starts at `k0`.  KC: element (o, k) at base[o * ld + k]; else base[k * ld + o].
template <bool KC>
__device__ __forceinline__ void gemm_load_tile(const float* __restrict__ base, int64_t ld, int o0, int k0, int O, int K,
                                               GemmStage& st) {
  const int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = t + i * kGemmThreads;
    if constexpr (KC) {
      const int o = o0 + idx / 8;
      const int k = k0 + (idx % 8) * 4;
      const int oc = min(o, O - 1);  // rows past the edge are never stored
      st.v[i] = k < K ? *reinterpret_cast<const float4*>(base + static_cast<int64_t>(oc) * ld + k)
                      : make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
      const int k = k0 + idx / 32;
      const int o = o0 + (idx % 32) * 4;
      st.v[i] = (k < K && o < O) ? *reinterpret_cast<const float4*>(base + static_cast<int64_t>(k) * ld + o)
                                 : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
}

template <bool KC>
__device__ __forceinline__ void gemm_store_tile(float* __restrict__ lds, const GemmStage& st) {
  const int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = t + i * kGemmThreads;
    if constexpr (KC) {
      *reinterpret_cast<float4*>(lds + (idx / 8) * kKcStride + (idx % 8) * 4) = st.v[i];
    } else {
      *reinterpret_cast<float4*>(lds + (idx / 32) * kGemmBM + (idx % 32) * 4) = st.v[i];
    }
  }
}

// MFMA operand values of one 32-wide tile for one group of 8 k-values: lane (o = l % 32,
// h = l / 32) takes k = g*8 + h*4 + j for j = 0..3, so MFMA j of the group multiplies
// k in {g*8 + j, g*8 + 4 + j}: each k is used exactly once, in an order that lets a
// k-contiguous operand be read with one 128-bit LDS load.
template <bool KC>
__device__ __forceinline__ void gemm_read_frag(const float* __restrict__ lds, int o_base, int g, float (&f)[4]) {
  const int lane = threadIdx.x % kWave;
  const int o = o_base + lane % 32;
  const int k = g * 8 + (lane / 32) * 4;
  if constexpr (KC) {
    const float4 r = *reinterpret_cast<const float4*>(lds + o * kKcStride + k);
    f[0] = r.x; f[1] = r.y; f[2] = r.z; f[3] = r.w;
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) f[j] = lds[(k + j) * kGemmBM + o];
  }
}

template <bool A_KC, bool B_KC, bool HAS_BIAS>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_f32_mfma_kernel(
    const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ bias, float* __restrict__ C,
    int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int64_t bsa, int64_t bsb, int64_t bsc, int tiles_m,
    int tiles_n, int total_work, GemmEpilogue<float> ep_in) {
  __shared__ __attribute__((aligned(16))) float lds_a[kGemmBM * kKcStride];
  __shared__ __attribute__((aligned(16))) float lds_b[kGemmBN * kKcStride];

  const int tiles = tiles_m * tiles_n;
  const float* const A_in = A;
  const float* const B_in = B;
  float* const C_in = C;
  // The grid holds at most the workgroups that are resident at once; each takes output tiles
  // work, work + gridDim.x, ...  Workgroups that share operand slabs then start every tile
  // together, which keeps their fetches of the shared rows close in time.
  for (int work = blockIdx.x; work < total_work; work += gridDim.x) {
  const int batch = work / tiles;
  int tm, tn;
  gemm_tile_of_block(work % tiles, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * kGemmBM;
  const int n0 = tn * kGemmBN;
  A = A_in + batch * bsa;
  B = B_in + batch * bsb;
  C = C_in + batch * bsc;
  GemmEpilogue<float> ep = ep_in;
  if (ep.residual) ep.residual += batch * bsc;
  if (ep.relu_mask) ep.relu_mask += batch * bsc;

  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int wm = (wave / 2) * 64;
  const int wn = (wave % 2) * 64;

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  GemmStage sa, sb;
  gemm_load_tile<A_KC>(A, lda, m0, 0, M, K, sa);
  gemm_load_tile<B_KC>(B, ldb, n0, 0, N, K, sb);

  for (int k0 = 0; k0 < K; k0 += kGemmBK) {
    gemm_store_tile<A_KC>(lds_a, sa);
    gemm_store_tile<B_KC>(lds_b, sb);
    __syncthreads();
    if (k0 + kGemmBK < K) {
      gemm_load_tile<A_KC>(A, lda, m0, k0 + kGemmBK, M, K, sa);
      gemm_load_tile<B_KC>(B, ldb, n0, k0 + kGemmBK, N, K, sb);
    }
#pragma unroll
    for (int g = 0; g < kGemmBK / 8; ++g) {
      float fa[2][4], fb[2][4];
      gemm_read_frag<A_KC>(lds_a, wm, g, fa[0]);
      gemm_read_frag<A_KC>(lds_a, wm + 32, g, fa[1]);
      gemm_read_frag<B_KC>(lds_b, wn, g, fb[0]);
      gemm_read_frag<B_KC>(lds_b, wn + 32, g, fb[1]);
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
          for (int tj = 0; tj < 2; ++tj)
            acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[ti][j], fb[tj][j], acc[ti][tj], 0, 0, 0);
    }
    __syncthreads();
  }

  // Accumulator element r of a lane is row (r/4)*8 + (lane/32)*4 + r%4, column lane%32.
#pragma unroll
  for (int ti = 0; ti < 2; ++ti)
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      const int col = n0 + wn + tj * 32 + lane % 32;
      if (col >= N) continue;
      const float bv = HAS_BIAS ? bias[col] : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm + ti * 32 + (r / 4) * 8 + (lane / 32) * 4 + (r % 4);
        if (row < M) {
          const int64_t at = static_cast<int64_t>(row) * ldc + col;
          C[at] = gemm_finish<float>(acc[ti][tj][r] + bv, ep, at);
        }
      }
    }
  }  // tiles of this workgroup
}

// ------------------------------------------------------------------------------------
// Any strides, any of the three float types: 64x64 tile, 256 threads, 4x4 outputs per
// thread, fp32 FMA.  The path for operands the MFMA kernels cannot take (unaligned
// leading dimensions, both strides non-unit, skinny edge shapes).
//   A element (m, k) at A[m * sam + k * sak];  B element (k, n) at B[k * sbk + n * sbn].
// ------------------------------------------------------------------------------------

template <typename T, bool HAS_BIAS>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const T* __restrict__ A, const T* __restrict__ B,
                                                           const T* __restrict__ bias, T* __restrict__ C, int M, int N,
                                                           int K, int64_t sam, int64_t sak, int64_t sbk, int64_t sbn,
                                                           int64_t ldc, int64_t bsa, int64_t bsb, int64_t bsc,
                                                           GemmEpilogue<T> ep) {
  constexpr int TM = 64, TN = 64, TK = 16;
  __shared__ float as[TK][TM + 1];
  __shared__ float bs[TK][TN + 1];
  const int batch = blockIdx.z;
  A += batch * bsa;
  B += batch * bsb;
  C += batch * bsc;
  if (ep.residual) ep.residual += batch * bsc;
  if (ep.relu_mask) ep.relu_mask += batch * bsc;
  const int m0 = blockIdx.y * TM;
  const int n0 = blockIdx.x * TN;
  const int tx = threadIdx.x % 16;
  const int ty = threadIdx.x / 16;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += TK) {
    for (int idx = threadIdx.x; idx < TM * TK; idx += 256) {
      // Walk the contiguous dimension fastest for whichever stride is 1.
      int m, k;
      if (sak == 1) { k = idx % TK; m = idx / TK; } else { m = idx % TM; k = idx / TM; }
      const int gm = m0 + m, gk = k0 + k;
      as[k][m] = (gm < M && gk < K) ? to_float(A[gm * sam + gk * sak]) : 0.f;
    }
    for (int idx = threadIdx.x; idx < TN * TK; idx += 256) {
      int n, k;
      if (sbk == 1) { k = idx % TK; n = idx / TK; } else { n = idx % TN; k = idx / TN; }
      const int gn = n0 + n, gk = k0 + k;
      bs[k][n] = (gn < N && gk < K) ? to_float(B[gk * sbk + gn * sbn]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = as[k][ty + i * 16];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = bs[k][tx + j * 16];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gm = m0 + ty + i * 16, gn = n0 + tx + j * 16;
      if (gm < M && gn < N) {
        const float bv = HAS_BIAS ? to_float(bias[gn]) : 0.f;
        const int64_t at = static_cast<int64_t>(gm) * ldc + gn;
        C[at] = gemm_finish<T>(acc[i][j] + bv, ep, at);
      }
    }
}

}  // namespace mg

// ------------------------------------------------------------------------------------
// 16-bit storage (bf16, fp16) on v_mfma_f32_32x32x16: 128x128 output tile, K-chunks of 64,
// four waves in a 2x2 grid, each a 64x64 tile (2x2 accumulators), fp32 accumulation.
// Both operand tiles live in LDS as [row][k] with k contiguous, which is what the MFMA
// wants (8 consecutive k per lane).  A k-contiguous operand is copied as is; an
// m/n-contiguous operand is transposed on the way in: a thread loads 8 columns of two
// consecutive k rows and stores 8 dwords, each packing (k, k+1) for one column.
// SPLIT_K: a workgroup takes one K range (gemm_split_work) and fp32 partial tiles go to scratch
// (splits, M, N); gemm_splitk_reduce_kernel sums them in a fixed order.
// ------------------------------------------------------------------------------------

namespace mg {

typedef __bf16 gemm_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 gemm_f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 gemm_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 gemm_f16x2 __attribute__((ext_vector_type(2)));
typedef float gemm_f32x2 __attribute__((ext_vector_type(2)));

// Two fp32 values rounded to T (nearest even), the first in the low half.
template <typename T>
__device__ __forceinline__ uint32_t gemm16_pack2(float lo, float hi);
template <>
__device__ __forceinline__ uint32_t gemm16_pack2<bf16_t>(float lo, float hi) {
  return bf16_pack2_rne(lo, hi);
}
template <>
__device__ __forceinline__ uint32_t gemm16_pack2<f16_t>(float lo, float hi) {
  const gemm_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, gemm_f16x2));
}

template <typename T>
struct GemmMma16;
template <>
struct GemmMma16<bf16_t> {
  static __device__ __forceinline__ floatx16 run(uint4 a, uint4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(gemm_bf16x8, a), __builtin_bit_cast(gemm_bf16x8, b),
                                                   c, 0, 0, 0);
  }
};
template <>
struct GemmMma16<f16_t> {
  static __device__ __forceinline__ floatx16 run(uint4 a, uint4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(gemm_f16x8, a), __builtin_bit_cast(gemm_f16x8, b), c,
                                                  0, 0, 0);
  }
};

constexpr int kG16BK = 64;
constexpr int kG16Stride = kG16BK + 8;  // elements per LDS row: 144 bytes, 16-byte aligned, bank-spreading
// fp32 partial tiles of a product split along K: [K range][batch][tile_m][tile_n] tiles of
// 128 x 128 values, each stored as its four waves' accumulators,
//   [wave][ti][tj][g][lane][j]  =  row (wave / 2) * 64 + ti * 32 + g * 8 + (lane / 32) * 4 + j,
//                                  column (wave % 2) * 64 + tj * 32 + lane % 32
// of the tile.  Tiles are stored whole; rows and columns past the matrix hold whatever the
// clamped operand rows produced and are dropped by the reduction.
constexpr int kG16PartialTile = kGemmBM * kGemmBN;
constexpr int kGemmWideBN = 384;  // columns of the wide tile of linear_bwd_16bit_kernel
inline int64_t gemm16_partial_floats(int64_t M, int64_t N, int64_t batches, int64_t splits) {
  return splits * batches * ((M + kGemmBM - 1) / kGemmBM) * ((N + kGemmBN - 1) / kGemmBN) * kG16PartialTile;
}

struct Gemm16Stage {
  uint4 v[4];
};

// KC: element (o, k) at base[o * ld + k].  4 chunks of 8 k-values per thread.
// else: element (o, k) at base[k * ld + o].  2 tasks per thread, each two k rows x 8 o.
// RAGGED: leading dimension, extents or base address are not multiples of 8 elements, so
// each chunk is assembled from eight 2-byte loads with per-element bounds.
template <typename T>
__device__ __forceinline__ uint4 gemm16_gather8(const T* __restrict__ p, int valid) {
  const uint16_t* q = reinterpret_cast<const uint16_t*>(p);
  uint32_t w[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t lo = 2 * e < valid ? q[2 * e] : 0u;
    const uint32_t hi = 2 * e + 1 < valid ? q[2 * e + 1] : 0u;
    w[e] = lo | (hi << 16);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

template <typename T, bool KC, bool RAGGED>
__device__ __forceinline__ void gemm16_load(const T* __restrict__ base, int64_t ld, int o0, int k0, int O, int k_end,
                                            Gemm16Stage& st) {
  const int t = threadIdx.x;
  if constexpr (RAGGED && KC) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = t + i * kGemmThreads;
      const int o = min(o0 + idx / 8, O - 1);
      const int k = k0 + (idx % 8) * 8;
      st.v[i] = gemm16_gather8(base + static_cast<int64_t>(o) * ld + k, k_end - k);
    }
  } else if constexpr (RAGGED) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int idx = t + i * kGemmThreads;
      const int oc = idx % 16, kp = idx / 16;
      const int k = k0 + 2 * kp;
      const int o = o0 + oc * 8;
      st.v[2 * i] = gemm16_gather8(base + static_cast<int64_t>(k) * ld + o, k < k_end ? O - o : 0);
      st.v[2 * i + 1] = gemm16_gather8(base + static_cast<int64_t>(k + 1) * ld + o, k + 1 < k_end ? O - o : 0);
    }
  } else if constexpr (KC) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = t + i * kGemmThreads;
      const int o = min(o0 + idx / 8, O - 1);  // rows past the edge are never stored
      const int k = k0 + (idx % 8) * 8;
      st.v[i] = k < k_end ? *reinterpret_cast<const uint4*>(base + static_cast<int64_t>(o) * ld + k)
                          : make_uint4(0, 0, 0, 0);
    }
  } else {
    // 16 consecutive lanes read the 256 contiguous bytes of one k row: whole cache lines.
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int idx = t + i * kGemmThreads;
      const int oc = idx % 16, kp = idx / 16;
      const int k = k0 + 2 * kp;
      const int o = o0 + oc * 8;
      const bool o_ok = o < O;
      st.v[2 * i] = (o_ok && k < k_end) ? *reinterpret_cast<const uint4*>(base + static_cast<int64_t>(k) * ld + o)
                                        : make_uint4(0, 0, 0, 0);
      st.v[2 * i + 1] = (o_ok && k + 1 < k_end)
                            ? *reinterpret_cast<const uint4*>(base + static_cast<int64_t>(k + 1) * ld + o)
                            : make_uint4(0, 0, 0, 0);
    }
  }
}

template <bool KC>
__device__ __forceinline__ void gemm16_store(uint16_t* __restrict__ lds, const Gemm16Stage& st) {
  const int t = threadIdx.x;
  if constexpr (KC) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = t + i * kGemmThreads;
      *reinterpret_cast<uint4*>(lds + (idx / 8) * kG16Stride + (idx % 8) * 8) = st.v[i];
    }
  } else {
    uint32_t* lds32 = reinterpret_cast<uint32_t*>(lds);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int idx = t + i * kGemmThreads;
      const int oc = idx % 16, kp = idx / 16;
      const uint32_t a[4] = {st.v[2 * i].x, st.v[2 * i].y, st.v[2 * i].z, st.v[2 * i].w};
      const uint32_t b[4] = {st.v[2 * i + 1].x, st.v[2 * i + 1].y, st.v[2 * i + 1].z, st.v[2 * i + 1].w};
      // The 16-byte k group of a row is stored at group index (g ^ (row / 8) % 8): the 16
      // lanes that hold different 8-row blocks of the same k pair then hit different banks
      // (row stride 36 dwords is 4 mod 32, so 8-row blocks alone would all collide).
      uint32_t* dst = lds32 + (oc * 8) * (kG16Stride / 2) + (((kp / 4) ^ (oc & 7)) * 4 + kp % 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        dst[(2 * e) * (kG16Stride / 2)] = __builtin_amdgcn_perm(b[e], a[e], 0x05040100);
        dst[(2 * e + 1) * (kG16Stride / 2)] = __builtin_amdgcn_perm(b[e], a[e], 0x07060302);
      }
    }
  }
}

template <bool SWIZZLED>
__device__ __forceinline__ uint4 gemm16_frag(const uint16_t* __restrict__ lds, int o_base, int ks, int lane) {
  const int row = o_base + lane % 32;
  int g = ks * 2 + lane / 32;  // 16-byte k group
  if constexpr (SWIZZLED) g ^= (row >> 3) & 7;
  return *reinterpret_cast<const uint4*>(lds + row * kG16Stride + g * 8);
}

// Output of one 128x128 tile from the four waves' accumulators (wave tile 64x64 at (wm, wn)).
// The accumulators have lanes along n and registers along m, so a direct store writes
// 2-byte elements.  When rows of C can be written 16 bytes at a time, each wave instead
// transposes its tile through `mine`, 64 rows of kG16Stride elements of LDS that no wave
// reads any more, and stores eight elements per lane.  SPLIT_K: fp32 partial tiles go to
// partial[(split * batches + batch), M, N].
template <typename T, bool HAS_BIAS, bool SPLIT_K>
__device__ __forceinline__ void gemm16_write_tile(const floatx16 (&acc)[2][2], uint16_t* __restrict__ mine,
                                                  const T* __restrict__ bias, T* __restrict__ C,
                                                  float* __restrict__ partial, int M, int N, int64_t ldc, int64_t bsc,
                                                  int batch, int split, int batches, int m0, int n0, int wm, int wn,
                                                  int lane, const GemmEpilogue<T>& ep, bool partial_stream = false,
                                                  const float* bias_early = nullptr) {
  if constexpr (SPLIT_K) {
    // A K range's partial tile goes out as the accumulators lie in the registers: sixteen
    // unguarded 16-byte stores per thread, each a contiguous kilobyte of the wave
    // (see gemm16_partial_floats for the layout; gemm_splitk_reduce_block undoes it).
    const int tiles_n = (N + kGemmBN - 1) / kGemmBN, tiles_m = (M + kGemmBM - 1) / kGemmBM;
    const int col0 = n0 + wn;  // a multiple of 64; the workgroup's tile may span several partial tiles
    const int64_t tile_at = (static_cast<int64_t>(split) * batches + batch) * tiles_m * tiles_n +
                            static_cast<int64_t>(m0 / kGemmBM) * tiles_n + col0 / kGemmBN;
    float4* dst = reinterpret_cast<float4*>(partial) + tile_at * (kG16PartialTile / 4) +
                  ((wm / 64) * 2 + (col0 / 64) % 2) * 1024 + lane;
    if (partial_stream) {
#pragma unroll
      for (int ti = 0; ti < 2; ++ti)
#pragma unroll
        for (int tj = 0; tj < 2; ++tj)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const floatx4 v = {acc[ti][tj][4 * g], acc[ti][tj][4 * g + 1], acc[ti][tj][4 * g + 2], acc[ti][tj][4 * g + 3]};
            __builtin_nontemporal_store(v, reinterpret_cast<floatx4*>(dst + ((ti * 2 + tj) * 4 + g) * 64));
          }
      return;
    }
#pragma unroll
    for (int ti = 0; ti < 2; ++ti)
#pragma unroll
      for (int tj = 0; tj < 2; ++tj)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          dst[((ti * 2 + tj) * 4 + g) * 64] = make_float4(acc[ti][tj][4 * g], acc[ti][tj][4 * g + 1],
                                                          acc[ti][tj][4 * g + 2], acc[ti][tj][4 * g + 3]);
    return;
  } else {
    const bool wide_out = (N % 8 == 0) && (ldc % 8 == 0) && (bsc % 8 == 0) && (reinterpret_cast<uintptr_t>(C) % 16 == 0);
    if (wide_out) {
      // An accumulator holds one column and, per group of four registers, four consecutive
      // rows.  Two lanes with neighbouring columns swap packed pairs of rows, so that the even
      // lane holds (own, neighbour) of the first row of a pair and the odd lane (neighbour,
      // own) of the second: 32 four-byte LDS writes per thread instead of 64 two-byte ones,
      // and three VALU instructions per pair (convert, swap, byte select).
      const int odd = lane & 1;
      const uint32_t select = odd ? 0x03020706u : 0x05040100u;
      uint32_t* const base32 =
          reinterpret_cast<uint32_t*>(mine + ((lane / 32) * 4 + odd) * kG16Stride + (lane % 32 - odd));
      // (One copy of the loop per setting of the relu flag: inside the loop the flag would
      // cost two more instructions per value.)
      auto stage = [&](auto relu) {
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
          for (int tj = 0; tj < 2; ++tj) {
            float bv = 0.f;
            if constexpr (HAS_BIAS) {
              const int col = n0 + wn + tj * 32 + lane % 32;
              bv = bias_early ? bias_early[tj] : (col < N ? to_float(bias[col]) : 0.f);
            }
#pragma unroll
            for (int rp = 0; rp < 8; ++rp) {  // rows 2 rp and 2 rp + 1 of the sixteen
              float f0 = acc[ti][tj][2 * rp], f1 = acc[ti][tj][2 * rp + 1];
              if constexpr (HAS_BIAS) f0 += bv, f1 += bv;
              if constexpr (decltype(relu)::value) {
                f0 = f0 > 0.f ? f0 : 0.f;
                f1 = f1 > 0.f ? f1 : 0.f;
              }
              const uint32_t w = gemm16_pack2<T>(f0, f1);
              const uint32_t y = __builtin_amdgcn_update_dpp(w, w, kDppQuadXor1, 0xf, 0xf, false);
              const int rl = ti * 32 + (rp / 2) * 8 + (rp % 2) * 2;  // without the lane's own (lane / 32) * 4 + odd
              base32[(rl * kG16Stride + tj * 32) / 2] = __builtin_amdgcn_perm(y, w, select);
            }
          }
      };
      if (ep.relu) stage(std::true_type{});
      else stage(std::false_type{});
      __syncthreads();
      // Rows of the wave's 64 x 64 tile go out 16 bytes per lane, eight lanes to a row, eight
      // rows per store: one address per thread, stepped by eight rows.
      const int rl0 = lane / 8, ch = lane % 8;
      const int row0 = m0 + wm + rl0;
      const int col = n0 + wn + ch * 8;
      if (col >= N) return;
      const int64_t at0 = batch * bsc + static_cast<int64_t>(row0) * ldc + col;
      const int64_t step = 8 * ldc;
      const uint16_t* src = mine + rl0 * kG16Stride + ch * 8;
      const T* rbase = ep.residual;
      const T* mbase = ep.relu_mask;
      if (!rbase && !mbase) {
        T* dst = C + at0;
        uint4 v[8];  // all eight LDS reads first: their latencies overlap
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = *reinterpret_cast<const uint4*>(src + i * 8 * kG16Stride);
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (row0 + 8 * i < M) *reinterpret_cast<uint4*>(dst + i * step) = v[i];
        return;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (row0 + 8 * i >= M) break;
        const int64_t at = at0 + i * step;
        float v[8];
        VecIO<T, 8>::load(reinterpret_cast<const T*>(src + i * 8 * kG16Stride), v);
        if (mbase) {
          float mk[8];
          VecIO<T, 8>::load(mbase + at, mk);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = mk[e] > 0.f ? v[e] : 0.f;
        }
        if (rbase) {
          float rs[8];
          VecIO<T, 8>::load(rbase + at, rs);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += rs[e];
        }
        VecIO<T, 8>::store(C + at, v);
      }
      return;
    }
  }
#pragma unroll
  for (int ti = 0; ti < 2; ++ti)
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      const int col = n0 + wn + tj * 32 + lane % 32;
      if (col >= N) continue;
      const float bv = HAS_BIAS ? to_float(bias[col]) : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm + ti * 32 + (r / 4) * 8 + (lane / 32) * 4 + (r % 4);
        if (row < M) {
          const int64_t at = batch * bsc + static_cast<int64_t>(row) * ldc + col;
          C[at] = gemm_finish<T>(acc[ti][tj][r] + bv, ep, at);
        }
      }
    }
}

// What a product's output tile needs to continue as a LayerNorm backward (see gemm16_ln_bwd_tile).
template <typename T>
struct Gemm16LayerNormBwd {
  const T* x = nullptr;         // the LayerNorm's input, laid out like the product's output
  const T* gamma = nullptr;     // (cols)
  const float* mean = nullptr;  // (rows) saved by the forward
  const float* rstd = nullptr;
  float* part_g = nullptr;      // (row tiles, cols) partial column sums of dy * xhat and of dy
  float* part_b = nullptr;
};

// Output of a 128 x (64 WN) tile whose rows are whole rows of the result (N = 64 WN), when the
// result dY is only wanted as the upstream of a LayerNorm backward: the tile is staged in LDS
// as the rounded 16-bit values a store would have written, and the workgroup then computes,
// from LDS and the matching rows of the LayerNorm's input x,
//   dx = rstd (dY gamma - mean_n(dY gamma) - xhat mean_n(dY gamma xhat)),  xhat = (x - mean) rstd,
// written to C as round(dx) (+ the residual, as the separate kernels give it), and the tile's
// column sums of dY xhat and dY as one row of part_g / part_b.  dY itself never reaches memory.
// A lane owns 8 columns of rows rl0 + 8 i of its wave's 64 x 64 tile (the layout of the plain
// store); a row's sums go over the 8 lanes of its 64 columns by DPP and over the WN waves that
// share the row through LDS, in a fixed order, and the column sums over the 8 row lanes by
// shuffles and over the two row waves through LDS.  `free_lds` is LDS behind the waves' strips:
// 128 * WN * 8 bytes for the row sums and 2 * 64 * WN * 8 for the column sums.
template <typename T, int WN>
__device__ __forceinline__ void gemm16_ln_bwd_tile(const floatx16 (&acc)[2][2], uint16_t* __restrict__ mine,
                                                   float* __restrict__ free_lds, T* C, int M, int64_t ldc, int tile_m,
                                                   int m0, int wm, int wn, int lane, const T* residual,
                                                   const Gemm16LayerNormBwd<T>& ln) {  // residual may be C itself
  constexpr int COLS = 64 * WN;
  {  // the staging of gemm16_write_tile (no bias, no ReLU)
    const int odd = lane & 1;
    const uint32_t select = odd ? 0x03020706u : 0x05040100u;
    uint32_t* const base32 = reinterpret_cast<uint32_t*>(mine + ((lane / 32) * 4 + odd) * kG16Stride + (lane % 32 - odd));
#pragma unroll
    for (int ti = 0; ti < 2; ++ti)
#pragma unroll
      for (int tj = 0; tj < 2; ++tj)
#pragma unroll
        for (int rp = 0; rp < 8; ++rp) {
          const uint32_t w = gemm16_pack2<T>(acc[ti][tj][2 * rp], acc[ti][tj][2 * rp + 1]);
          const uint32_t y = __builtin_amdgcn_update_dpp(w, w, kDppQuadXor1, 0xf, 0xf, false);
          const int rl = ti * 32 + (rp / 2) * 8 + (rp % 2) * 2;
          base32[(rl * kG16Stride + tj * 32) / 2] = __builtin_amdgcn_perm(y, w, select);
        }
  }
  float2* row_sums = reinterpret_cast<float2*>(free_lds);               // [128][WN]
  float* col_sums = free_lds + 128 * WN * 2;                             // [2 row waves][which][COLS]
  const int rl0 = lane / 8, ch = lane % 8;
  const int col = wn + ch * 8;
  const uint16_t* src = mine + rl0 * kG16Stride + ch * 8;
  float gam[8];
  VecIO<T, 8>::load(ln.gamma + col, gam);
  uint4 xraw[8], rraw[8];
  float mu[8], rs[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = min(m0 + wm + rl0 + 8 * i, M - 1);  // rows past the end: computed, never stored or summed
    const int64_t at = static_cast<int64_t>(row) * ldc + col;
    xraw[i] = *reinterpret_cast<const uint4*>(ln.x + at);
    rraw[i] = residual ? *reinterpret_cast<const uint4*>(residual + at) : make_uint4(0, 0, 0, 0);
    mu[i] = ln.mean[row];
    rs[i] = ln.rstd[row];
  }
  __syncthreads();  // the strips are complete
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float dy[8], xv[8];
    VecIO<T, 8>::load(reinterpret_cast<const T*>(src + i * 8 * kG16Stride), dy);
    VecIO<T, 8>::load(reinterpret_cast<const T*>(&xraw[i]), xv);
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float xhat = (xv[e] - mu[i]) * rs[i];
      const float dyg = dy[e] * gam[e];
      s0 += dyg;
      s1 += dyg * xhat;
    }
    s0 += dpp_move<kDppQuadXor1>(s0);
    s1 += dpp_move<kDppQuadXor1>(s1);
    s0 += dpp_move<kDppQuadXor2>(s0);
    s1 += dpp_move<kDppQuadXor2>(s1);
    s0 += dpp_move<kDppRowHalfMirror>(s0);
    s1 += dpp_move<kDppRowHalfMirror>(s1);
    if (ch == 0) row_sums[(wm + rl0 + 8 * i) * WN + wn / 64] = make_float2(s0, s1);
  }
  __syncthreads();
  const float inv_n = 1.0f / static_cast<float>(COLS);
  float acc_g[8], acc_b[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc_g[e] = acc_b[e] = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = m0 + wm + rl0 + 8 * i;
    float c1 = 0.f, c2 = 0.f;
#pragma unroll
    for (int w = 0; w < WN; ++w) {
      const float2 p = row_sums[(wm + rl0 + 8 * i) * WN + w];
      c1 += p.x;
      c2 += p.y;
    }
    c1 *= inv_n;
    c2 *= inv_n;
    float dy[8], xv[8], rv[8], out[8];
    VecIO<T, 8>::load(reinterpret_cast<const T*>(src + i * 8 * kG16Stride), dy);
    VecIO<T, 8>::load(reinterpret_cast<const T*>(&xraw[i]), xv);
    VecIO<T, 8>::load(reinterpret_cast<const T*>(&rraw[i]), rv);
    const bool ok = row < M;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float xhat = (xv[e] - mu[i]) * rs[i];
      const float d = ok ? dy[e] : 0.f;
      out[e] = rs[i] * (d * gam[e] - c1 - xhat * c2);
      acc_g[e] += d * xhat;
      acc_b[e] += d;
    }
    if (residual) {
      // round(gradient) + residual: a plain addition, as the separate add performs it
#pragma clang fp contract(off)
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = to_float(from_float<T>(out[e])) + rv[e];
    }
    if (ok) VecIO<T, 8>::store(C + static_cast<int64_t>(row) * ldc + col, out);
  }
  // column sums over the wave's 64 rows: the 8 lanes with this lane's columns
#pragma unroll
  for (int e = 0; e < 8; ++e) {
#pragma unroll
    for (int w = 8; w < kWave; w *= 2) {
      acc_g[e] += __shfl_xor(acc_g[e], w);
      acc_b[e] += __shfl_xor(acc_b[e], w);
    }
  }
  if (rl0 == 0) {
    float* mine_g = col_sums + (wm / 64) * 2 * COLS + col;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      mine_g[e] = acc_g[e];
      mine_g[COLS + e] = acc_b[e];
    }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < COLS; c += blockDim.x) {
    ln.part_g[static_cast<int64_t>(tile_m) * COLS + c] = col_sums[c] + col_sums[2 * COLS + c];
    ln.part_b[static_cast<int64_t>(tile_m) * COLS + c] = col_sums[COLS + c] + col_sums[3 * COLS + c];
  }
}

template <typename T, bool A_KC, bool B_KC, bool HAS_BIAS, bool SPLIT_K, bool RAGGED>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_16bit_mfma_kernel(
    const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ bias, T* __restrict__ C,
    float* __restrict__ partial, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int64_t bsa, int64_t bsb,
    int64_t bsc, int tiles_m, int tiles_n, int k_per_split, int splits, int batches, GemmEpilogue<T> ep) {
  __shared__ __attribute__((aligned(16))) uint16_t lds_a[kGemmBM * kG16Stride];
  __shared__ __attribute__((aligned(16))) uint16_t lds_b[kGemmBN * kG16Stride];

  const int tiles = tiles_m * tiles_n;
  // Split along K: see gemm_split_work.  Otherwise the batch index is folded into the tile id.
  int batch = blockIdx.x / tiles, tile = blockIdx.x % tiles, split = 0;
  if constexpr (SPLIT_K) {
    if (!gemm_split_work(blockIdx.x, tiles, splits, batches, tile, split, batch)) return;
  }
  int tm, tn;
  gemm_tile_of_block(tile, tiles_m, tiles_n, tm, tn, !SPLIT_K);
  const int m0 = tm * kGemmBM;
  const int n0 = tn * kGemmBN;
  A += batch * bsa;
  B += batch * bsb;
  const int k_begin = SPLIT_K ? split * k_per_split : 0;
  const int k_end = SPLIT_K ? min(K, k_begin + k_per_split) : K;

  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int wm = (wave / 2) * 64;
  const int wn = (wave % 2) * 64;

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // The lane's two bias values, requested ahead of the first tiles (a load in the epilogue
  // would be waited for by every tile with nothing to overlap it).
  float bias_v[2] = {0.f, 0.f};
  if constexpr (HAS_BIAS && !SPLIT_K) {
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      const int col = n0 + wn + tj * 32 + lane % 32;
      bias_v[tj] = col < N ? to_float(bias[col]) : 0.f;
    }
  }
  Gemm16Stage sa, sb;
  gemm16_load<T, A_KC, RAGGED>(A, lda, m0, k_begin, M, k_end, sa);
  gemm16_load<T, B_KC, RAGGED>(B, ldb, n0, k_begin, N, k_end, sb);

  for (int k0 = k_begin; k0 < k_end; k0 += kG16BK) {
    gemm16_store<A_KC>(lds_a, sa);
    gemm16_store<B_KC>(lds_b, sb);
    __syncthreads();
    if (k0 + kG16BK < k_end) {
      gemm16_load<T, A_KC, RAGGED>(A, lda, m0, k0 + kG16BK, M, k_end, sa);
      gemm16_load<T, B_KC, RAGGED>(B, ldb, n0, k0 + kG16BK, N, k_end, sb);
    }
#pragma unroll
    for (int ks = 0; ks < kG16BK / 16; ++ks) {
      const uint4 fa0 = gemm16_frag<!A_KC>(lds_a, wm, ks, lane);
      const uint4 fa1 = gemm16_frag<!A_KC>(lds_a, wm + 32, ks, lane);
      const uint4 fb0 = gemm16_frag<!B_KC>(lds_b, wn, ks, lane);
      const uint4 fb1 = gemm16_frag<!B_KC>(lds_b, wn + 32, ks, lane);
      acc[0][0] = GemmMma16<T>::run(fa0, fb0, acc[0][0]);
      acc[0][1] = GemmMma16<T>::run(fa0, fb1, acc[0][1]);
      acc[1][0] = GemmMma16<T>::run(fa1, fb0, acc[1][0]);
      acc[1][1] = GemmMma16<T>::run(fa1, fb1, acc[1][1]);
    }
    __syncthreads();
  }

  uint16_t* mine = (wave < 2 ? lds_a : lds_b) + (wave % 2) * 64 * kG16Stride;  // staging memory, idle now
  gemm16_write_tile<T, HAS_BIAS, SPLIT_K>(acc, mine, bias, C, partial, M, N, ldc, bsc, batch,
                                          split, SPLIT_K ? batches : 1,
                                          m0, n0, wm, wn, lane, ep, false, HAS_BIAS && !SPLIT_K ? bias_v : nullptr);
}

// ------------------------------------------------------------------------------------
// The same product with the tiles copied global memory -> LDS by the memory pipeline itself
// (`global_load_lds_dwordx4`: every lane names a 16-byte source, the wave's 64 chunks land
// back to back at an LDS address common to the wave), NSTAGE k-steps deep.  No registers
// hold data in flight, so several steps' loads are outstanding while one step is multiplied:
// what short-K products at a few hundred FLOP per byte need, being bound by memory latency
// and not by the matrix cores.  Operands as above, all extents and strides multiples of 8
// elements, K (and every K split) a multiple of 64.
//
// LDS image of one operand's step, chosen per 16-byte chunk by which source chunk each lane
// names (64 banks of four bytes; a 128-bit read is served 16 lanes per clock):
//   k-contiguous, 64 k per step: [128 rows][8 chunks], chunk c of row r at position
//     c ^ (r/2 % 8), with 32 k per step [128 rows][4 chunks] and c ^ (r/4 % 4): the sixteen
//     consecutive rows of a fragment read then hit sixteen different 16-byte bank groups
//     (timed on the device: 18.5-18.7 clocks per read with four waves reading, as for
//     consecutive addresses; 32 with c ^ (r % 8));
//   otherwise: [k][16 chunks of 8 rows], chunk c of k-row kk at position
//     c ^ gemm16_tr_swizzle(kk), read with `ds_read_b64_tr_b16` (within 16 lanes, lane i supplies
//     the four elements 4*i .. 4*i+3 of a 4 x 16 block and receives column i), which turns
//     four k-rows of 16 consecutive rows into each lane's four consecutive k.
// ------------------------------------------------------------------------------------

typedef short gemm_i16x4 __attribute__((ext_vector_type(4)));

// Where 16-byte chunk c of k-row kk of an m/n-contiguous operand sits in its LDS row:
// c ^ swizzle(kk).  A k-row is 256 or 512 bytes, a whole number of trips round the 64 banks,
// so without it every k-row would start on bank 0.  A transposing read takes 32 bytes of each
// of four k-rows (kk % 4 = 0..3) per sixteen lanes: 4 * (kk % 4) puts those on four different
// 32-byte bank groups that leave the neighbouring sixteen lanes' groups (chunk + 2) free, and
// 2 * (kk / 8 % 2) moves the upper half-wave (k-rows + 8) onto the remaining groups, so that
// whichever 32 lanes the LDS serves together touch every bank once.  (With c ^ 2 * (kk % 4),
// two sixteen-lane groups shared their bank groups: 43 % of the LDS cycles of the Linear
// backward kernel were conflict cycles.)
__device__ __forceinline__ constexpr int gemm16_tr_swizzle(int kk) { return 4 * (kk % 4) ^ 2 * ((kk / 8) % 2); }

// Copying one k-step of an operand of ROWS rows in a workgroup of NW waves: the waves that
// take part (all of them, unless the step has fewer kilobytes than the workgroup has waves)
// and the 16-byte requests of each of their threads.
constexpr int gemm16_pipe_waves(int rows, int bk, int nw) {
  const int kb = rows * bk * 2 / 1024;
  int w = kb < nw ? kb : nw;
  while (kb % w) --w;  // every taking wave the same number of kilobytes
  return w;
}
constexpr int gemm16_pipe_requests(int rows, int bk, int nw) {
  return rows * bk * 2 / 16 / (gemm16_pipe_waves(rows, bk, nw) * 64);
}

// The 16-byte source chunks this thread names for every k-step of one operand of ROWS rows,
// as element offsets from the operand's (batch, k_begin) origin; they advance by BK
// (k-contiguous) or BK * ld per step.
template <bool KC, int BK, int ROWS, int NW>  // NW: the waves that take part in this operand's copy
__device__ __forceinline__ void gemm16_pipe_sources(int64_t ld, int o0, int O,
                                                    int64_t (&src)[gemm16_pipe_requests(ROWS, BK, NW)]) {
  constexpr int CPR = BK / 8;     // chunks per k-contiguous row
  constexpr int CPK = ROWS / 8;   // chunks per k-row of the other image
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
#pragma unroll
  for (int i = 0; i < gemm16_pipe_requests(ROWS, BK, NW); ++i) {
    const int slot = (i * NW + wave) * kWave + lane;  // 16-byte position in the LDS image
    if constexpr (KC) {
      const int r = slot / CPR, c = (slot % CPR) ^ ((r / (16 / CPR)) % CPR);
      src[i] = static_cast<int64_t>(min(o0 + r, O - 1)) * ld + c * 8;  // rows past the edge are never stored
    } else {
      const int kk = slot / CPK, c = (slot % CPK) ^ gemm16_tr_swizzle(kk);
      const int o = o0 + c * 8;
      src[i] = static_cast<int64_t>(kk) * ld + (o < O ? o : o0);
    }
  }
}

// Written as assembly on purpose.  Through the compiler's builtin for this instruction every
// later LDS read of a kind whose aliasing it cannot judge (the transposing reads here) gets a
// wait for *all* outstanding copies, the younger steps' included, which would undo the
// pipeline; the waits are placed by hand in the kernel instead (MG_WAIT_VMCNT).  m0 (the
// wave's LDS destination) is written here and used by nothing else in these kernels.
template <int NI, int NW>
__device__ __forceinline__ void gemm16_pipe_issue(const uint16_t* base, const int64_t* src, char* lds_step) {
  using lds_ptr = __attribute__((address_space(3))) char*;
  const int wave = threadIdx.x / kWave;
  const unsigned dst = static_cast<unsigned>(reinterpret_cast<uintptr_t>((lds_ptr)lds_step)) + wave * 1024;
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const unsigned dst_i = __builtin_amdgcn_readfirstlane(dst + i * NW * 1024);
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst_i), "v"(base + src[i]) : "memory");
  }
}

// MFMA operand fragment: row o_base + lane % 32, k = ks * 16 + (lane / 32) * 8 .. + 7.
template <bool KC, int BK, int ROWS>
__device__ __forceinline__ uint4 gemm16_pipe_frag(const char* __restrict__ lds_step, int o_base, int ks, int lane) {
  if constexpr (KC) {
    constexpr int CPR = BK / 8;
    const int r = o_base + lane % 32;
    const int g = ks * 2 + lane / 32;
    return *reinterpret_cast<const uint4*>(lds_step + r * (BK * 2) + ((g ^ ((r / (16 / CPR)) % CPR)) * 16));
  } else {
    const int o = o_base + ((lane / 16) % 2) * 16 + 4 * (lane % 4);  // first of the 4 rows this lane supplies
    const int kq = (lane % 16) / 4;                                 // its k-row within a group of 4
    const int kk = ks * 16 + (lane / 32) * 8 + kq;
    const char* at = lds_step + kk * (ROWS * 2) + (((o / 8) ^ gemm16_tr_swizzle(kk)) * 16) + (o % 8) * 2;
    using lds_i16x4 = __attribute__((address_space(3))) gemm_i16x4;
    const gemm_i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        reinterpret_cast<lds_i16x4*>(reinterpret_cast<uintptr_t>(at)));
    const gemm_i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        reinterpret_cast<lds_i16x4*>(reinterpret_cast<uintptr_t>(at + 4 * (ROWS * 2))));
    uint2 l = __builtin_bit_cast(uint2, lo), h = __builtin_bit_cast(uint2, hi);
    return make_uint4(l.x, l.y, h.x, h.y);
  }
}

// s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt in bits 3:0 and
// 15:14, expcnt 6:4 and lgkmcnt 11:8 left at "no wait").
#define MG_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | 0x0f70)

// LDS of the pipelined kernel (TM = rows of the A tile: 128 with four waves, 256 with eight) and
// the workgroups that fit a CU, by LDS (160 KB) and by the register file.
constexpr int gemm16_pipe_lds_bytes(int bk, int nstage, int tm, int tn = 128) {
  const int stages = nstage * (tm + tn) * bk * 2;
  const int out = (tm / 64) * (tn / 64) * 64 * kG16Stride * 2;  // every wave transposes its output tile here
  return stages > out ? stages : out;
}
constexpr int gemm16_pipe_occupancy(int bk, int nstage, int tm, int tn = 128) {
  const int by_lds = 160 * 1024 / gemm16_pipe_lds_bytes(bk, nstage, tm, tn);
  const int by_regs = 16 / ((tm / 64) * (tn / 64));  // four waves per SIMD at most
  return by_lds < 1 ? 1 : (by_lds > by_regs ? by_regs : by_lds);
}

// One product's arguments, as the kernels below take them.
template <typename T>
struct Gemm16Problem {
  const T* A;
  const T* B;
  const T* bias;
  T* C;
  float* partial;
  int M, N, K;
  int64_t lda, ldb, ldc, bsa, bsb, bsc;
  int tiles_m, tiles_n, k_per_split, splits, batches;
  GemmEpilogue<T> ep;
  // Split along K with an m-contiguous A only (dW = dY^T X): when set, the workgroups of the
  // first tile column also sum their A tiles over k, i.e. dY over its rows, and leave one
  // partial row of the bias gradient per K range at colsum_part[split * M + m].
  float* colsum_part = nullptr;
  // The partial tiles are read back much later (their sum is deferred to the end of a training
  // step): store them past the caches.
  bool partial_stream = false;
  // The output continues as a LayerNorm backward inside the launch (gemm16_pipe_block<.., LN_BWD>).
  Gemm16LayerNormBwd<T> ln;
};

// The work of workgroup `bid` of a launch for one product; `lds` is the workgroup's
// gemm16_pipe_lds_bytes(BK, NSTAGE, TM, TN) bytes, aligned to 1024.  The output tile is
// TM x TN, (TM / 64) x (TN / 64) waves with 64 x 64 each; pr.tiles_n counts tiles of TN columns.
template <typename T, bool A_KC, bool B_KC, bool HAS_BIAS, bool SPLIT_K, int BK, int NSTAGE, int TM = 128,
          int TN = kGemmBN, bool LN_BWD = false>
__device__ __forceinline__ void gemm16_pipe_block(char* lds, int bid, const Gemm16Problem<T>& pr) {
  static_assert(NSTAGE >= 2 && NSTAGE <= 4 && (BK == 32 || BK == 64) && (TM == 128 || TM == 256), "stages");
  static_assert(TN % 128 == 0 && (!SPLIT_K || TM == 128), "partial tiles are 128 x 128");
  // The host cuts K ranges and checks K in units of kG16BK: every range is then whole steps of BK.
  static_assert(kG16BK % BK == 0, "K ranges are multiples of kG16BK, which must be whole steps");
  constexpr int WN = TN / 64;                                 // waves side by side
  constexpr int NW = (TM / 64) * WN;
  constexpr int NWA = gemm16_pipe_waves(TM, BK, NW), NWB = gemm16_pipe_waves(TN, BK, NW);  // waves that copy A, B
  constexpr int NIA = gemm16_pipe_requests(TM, BK, NW);       // copy requests per thread and step
  constexpr int NIB = gemm16_pipe_requests(TN, BK, NW);
  constexpr int OPA = TM * BK * 2, OPB = TN * BK * 2;         // bytes of an operand's step
  constexpr int OP = OPA + OPB;
  const T* __restrict__ A = pr.A;
  const T* __restrict__ B = pr.B;
  const T* __restrict__ bias = pr.bias;
  T* __restrict__ C = pr.C;
  float* __restrict__ partial = pr.partial;
  const int M = pr.M, N = pr.N, K = pr.K;
  const int64_t lda = pr.lda, ldb = pr.ldb, ldc = pr.ldc, bsa = pr.bsa, bsb = pr.bsb, bsc = pr.bsc;
  const int tiles_m = pr.tiles_m, tiles_n = pr.tiles_n, k_per_split = pr.k_per_split, splits = pr.splits,
            batches = pr.batches;
  const GemmEpilogue<T> ep = pr.ep;

  const int tiles = tiles_m * tiles_n;
  int batch = bid / tiles, tile = bid % tiles, split = 0;
  if constexpr (SPLIT_K) {
    if (!gemm_split_work(bid, tiles, splits, batches, tile, split, batch)) return;
  }
  int tm, tn;
  gemm_tile_of_block(tile, tiles_m, tiles_n, tm, tn, !SPLIT_K);
  const int m0 = tm * TM;
  const int n0 = tn * TN;
  const int k_begin = SPLIT_K ? split * k_per_split : 0;
  const int k_end = SPLIT_K ? min(K, k_begin + k_per_split) : K;
  const int steps = (k_end - k_begin) / BK;
  A += batch * bsa + (A_KC ? static_cast<int64_t>(k_begin) : k_begin * lda);
  B += batch * bsb + (B_KC ? static_cast<int64_t>(k_begin) : k_begin * ldb);
  const int64_t a_step = A_KC ? BK : BK * lda;
  const int64_t b_step = B_KC ? BK : BK * ldb;

  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int wm = (wave / WN) * 64;
  const int wn = (wave % WN) * 64;
  // Waves that copy fewer requests per step have fewer outstanding at the waits below.
  const bool copies_a = NWA == NW || wave < NWA, copies_b = NWB == NW || wave < NWB;
  const int per_step = (copies_a ? NIA : 0) + (copies_b ? NIB : 0);

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Column sums of the A tiles (see Gemm16Problem::colsum_part): a thread of the first four
  // waves takes one 16-byte chunk (8 of the tile's 128 m) of every 16th k-row.
  constexpr bool CAN_COLSUM = SPLIT_K && !A_KC && TM == 128;
  const bool colsum = CAN_COLSUM && pr.colsum_part != nullptr && tn == 0;
  const bool cs_thread = threadIdx.x < 256;
  const int cs_chunk = threadIdx.x % 16, cs_row = threadIdx.x / 16;
  float cs_acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) cs_acc[e] = 0.f;

  const uint16_t* a16 = reinterpret_cast<const uint16_t*>(A);
  const uint16_t* b16 = reinterpret_cast<const uint16_t*>(B);
  int64_t src_a[NIA], src_b[NIB];
  gemm16_pipe_sources<A_KC, BK, TM, NWA>(lda, m0, M, src_a);
  gemm16_pipe_sources<B_KC, BK, TN, NWB>(ldb, n0, N, src_b);
  auto request = [&](int step, int copy) {
    if (copies_a) gemm16_pipe_issue<NIA, NWA>(a16 + step * a_step, src_a, lds + copy * OP);
    if (copies_b) gemm16_pipe_issue<NIB, NWB>(b16 + step * b_step, src_b, lds + copy * OP + OPA);
  };

  // The lane's two bias values are requested before the tiles and are in their registers when
  // the first step's tiles are (the empty asm puts the compiler's wait here, where the first
  // iteration waits anyway): fetched in the epilogue, every tile ended on an exposed load, 4-10 us
  // of a 30-40 us product at 16384 rows.
  float bias_v[2] = {0.f, 0.f};
  if constexpr (HAS_BIAS && !SPLIT_K) {
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
      const int col = n0 + wn + tj * 32 + lane % 32;
      bias_v[tj] = col < N ? to_float(bias[col]) : 0.f;
    }
  }
  // Steps 0 .. NSTAGE-2 are requested up front; iteration `it` then waits for step `it`
  // (its own NIA + NIB requests; the barrier covers the other waves'), requests step
  // it + NSTAGE - 1 into the copy that step it - 1 was just multiplied from, and multiplies.
#pragma unroll
  for (int s = 0; s < NSTAGE - 1; ++s)
    if (s < steps) request(s, s);
  if constexpr (HAS_BIAS && !SPLIT_K) asm volatile("" : "+v"(bias_v[0]), "+v"(bias_v[1]));
  int cur = 0, nxt = NSTAGE - 1;
  for (int it = 0; it < steps; ++it) {
    // all but the NSTAGE - 2 younger steps' requests
    if (it + NSTAGE - 2 >= steps || NSTAGE == 2) MG_WAIT_VMCNT(0);
    else if (per_step == NIA + NIB) MG_WAIT_VMCNT((NIA + NIB) * (NSTAGE - 2));
    else if (per_step == NIB) MG_WAIT_VMCNT(NIB * (NSTAGE - 2));
    else if (per_step == NIA) MG_WAIT_VMCNT(NIA * (NSTAGE - 2));
    // A plain barrier: __syncthreads() carries a fence that waits for every outstanding
    // copy into LDS, the younger steps' included.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (it + NSTAGE - 1 < steps) request(it + NSTAGE - 1, nxt);
    const char* la = lds + cur * OP;
    const char* lb = la + OPA;
    if constexpr (CAN_COLSUM) {
      if (colsum && cs_thread) {
#pragma unroll
        for (int j = 0; j < BK / 16; ++j) {
          const int kk = cs_row + 16 * j;
          float v[8];
          VecIO<T, 8>::load(reinterpret_cast<const T*>(la + kk * (TM * 2) + ((cs_chunk ^ gemm16_tr_swizzle(kk)) * 16)), v);
#pragma unroll
          for (int e = 0; e < 8; ++e) cs_acc[e] += v[e];
        }
      }
    }
    // The fragments of k-slice ks + 1 are requested before the products of slice ks, so
    // their LDS latency runs under four MFMAs.
    uint4 fa[2][2], fb[2][2];
    fa[0][0] = gemm16_pipe_frag<A_KC, BK, TM>(la, wm, 0, lane);
    fa[0][1] = gemm16_pipe_frag<A_KC, BK, TM>(la, wm + 32, 0, lane);
    fb[0][0] = gemm16_pipe_frag<B_KC, BK, TN>(lb, wn, 0, lane);
    fb[0][1] = gemm16_pipe_frag<B_KC, BK, TN>(lb, wn + 32, 0, lane);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int c = ks % 2, n = c ^ 1;
      if (ks + 1 < BK / 16) {
        fa[n][0] = gemm16_pipe_frag<A_KC, BK, TM>(la, wm, ks + 1, lane);
        fa[n][1] = gemm16_pipe_frag<A_KC, BK, TM>(la, wm + 32, ks + 1, lane);
        fb[n][0] = gemm16_pipe_frag<B_KC, BK, TN>(lb, wn, ks + 1, lane);
        fb[n][1] = gemm16_pipe_frag<B_KC, BK, TN>(lb, wn + 32, ks + 1, lane);
      }
      acc[0][0] = GemmMma16<T>::run(fa[c][0], fb[c][0], acc[0][0]);
      acc[0][1] = GemmMma16<T>::run(fa[c][0], fb[c][1], acc[0][1]);
      acc[1][0] = GemmMma16<T>::run(fa[c][1], fb[c][0], acc[1][0]);
      acc[1][1] = GemmMma16<T>::run(fa[c][1], fb[c][1], acc[1][1]);
    }
    cur = cur + 1 == NSTAGE ? 0 : cur + 1;
    nxt = nxt + 1 == NSTAGE ? 0 : nxt + 1;
  }
  __syncthreads();  // every wave is done with the staged tiles: their memory serves the output

  if constexpr (CAN_COLSUM) {
    if (colsum) {
      // sixteen threads hold sums for the same 8 columns (k-rows 0, 16, ... / 1, 17, ... / ...):
      // added in a fixed order through LDS, one thread per column
      constexpr int kPitch = 128 + 4;
      float* red = reinterpret_cast<float*>(lds);
      if (cs_thread) {
#pragma unroll
        for (int e = 0; e < 8; ++e) red[cs_row * kPitch + cs_chunk * 8 + e] = cs_acc[e];
      }
      __syncthreads();
      if (threadIdx.x < 128 && m0 + static_cast<int>(threadIdx.x) < M) {
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) sum += red[r * kPitch + threadIdx.x];
        pr.colsum_part[static_cast<int64_t>(split) * M + m0 + threadIdx.x] = sum;
      }
      __syncthreads();
    }
  }

  uint16_t* mine = reinterpret_cast<uint16_t*>(lds) + wave * 64 * kG16Stride;
  if constexpr (LN_BWD) {
    // whole rows per tile, and room behind the strips for the row and column sums
    static_assert(!SPLIT_K && !HAS_BIAS && TM == 128, "the LayerNorm epilogue takes a plain 128-row tile");
    static_assert(gemm16_pipe_lds_bytes(BK, NSTAGE, TM, TN) >= NW * 64 * kG16Stride * 2 + 128 * WN * 8 + 2 * 64 * WN * 8,
                  "LDS behind the output strips");
    float* free_lds = reinterpret_cast<float*>(lds + NW * 64 * kG16Stride * 2);
    gemm16_ln_bwd_tile<T, WN>(acc, mine, free_lds, C + batch * bsc, M, ldc, tm, m0, wm, wn, lane, ep.residual, pr.ln);
  } else {
    gemm16_write_tile<T, HAS_BIAS, SPLIT_K>(acc, mine, bias, C, partial, M, N, ldc, bsc, batch,
                                            split, SPLIT_K ? batches : 1,
                                            m0, n0, wm, wn, lane, ep, pr.partial_stream,
                                            HAS_BIAS && !SPLIT_K ? bias_v : nullptr);
  }
}

template <typename T, bool A_KC, bool B_KC, bool HAS_BIAS, bool SPLIT_K, int BK, int NSTAGE, int TM = 128>
__global__ __launch_bounds__(TM * 2, gemm16_pipe_occupancy(BK, NSTAGE, TM)) void gemm_16bit_pipe_kernel(
    const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ bias, T* __restrict__ C,
    float* __restrict__ partial, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int64_t bsa, int64_t bsb,
    int64_t bsc, int tiles_m, int tiles_n, int k_per_split, int splits, int batches, GemmEpilogue<T> ep) {
  __shared__ __attribute__((aligned(1024))) char lds[gemm16_pipe_lds_bytes(BK, NSTAGE, TM)];
  const Gemm16Problem<T> pr{A, B, bias, C, partial, M, N, K, lda, ldb, ldc, bsa, bsb, bsc,
                            tiles_m, tiles_n, k_per_split, splits, batches, ep};
  gemm16_pipe_block<T, A_KC, B_KC, HAS_BIAS, SPLIT_K, BK, NSTAGE, TM>(lds, blockIdx.x, pr);
}

// ------------------------------------------------------------------------------------
// Large products: 256 x 256 output tile per workgroup of four waves, one wave per SIMD, each
// wave a 128 x 128 tile as 4 x 4 v_mfma_f32_32x32x16 accumulators (256 accumulator registers
// of the 512 a lone wave may use).  A k-slice of 16 takes four A and four B fragments for
// sixteen MFMAs, i.e. half a kilobyte of LDS reads per MFMA where the 64 x 64 wave tile of
// the kernels above needs a whole one: with four SIMDs issuing MFMAs back to back those
// kernels ask the LDS for exactly its 128 bytes per clock, this one for half of that, and a
// 256 x 256 tile also halves the operand bytes a FLOP pulls through L2.  The price is one
// workgroup per CU: no second wave hides a wait, so the fragments of slice ks + 1 are read
// while slice ks is multiplied and the tiles are copied NSTAGE steps ahead.  Taken for
// products with at least one such tile per CU; tiles, copy and LDS images are those of
// gemm16_pipe_block, and so is the order of every sum (results are bit-identical).
// 8192^3 bf16 forward / dX / dW: 1.26 / 1.11 / 1.02 ms with 256 x 128 tiles of 64 x 64 wave
// tiles -> 1.06 / 0.95 / 0.89 ms; matrix pipe busy 64 % of the CU-busy cycles (44-49 % before).
// With the copies compiled out the same loop takes 0.79 / 0.73 / 0.70 ms, with the MFMAs
// compiled out 0.63-0.72 / 0.63 / 0.57-0.64 ms: the L2 -> LDS copy of 8.6 GB per launch is as
// long as the arithmetic and the two do not overlap fully.
// ------------------------------------------------------------------------------------
constexpr int kGemmBigT = 256;
constexpr int gemm16_big_lds_bytes(int bk, int nstage) {
  const int stages = nstage * 2 * kGemmBigT * bk * 2;
  const int out = 4 * 64 * kG16Stride * 2;
  return stages > out ? stages : out;
}

template <typename T, bool A_KC, bool B_KC, bool HAS_BIAS, int BK, int NSTAGE>
__global__ __launch_bounds__(256, 1) void gemm_16bit_big_kernel(
    const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ bias, T* __restrict__ C, int M, int N, int K,
    int64_t lda, int64_t ldb, int64_t ldc, int64_t bsa, int64_t bsb, int64_t bsc, int tiles_m, int tiles_n,
    GemmEpilogue<T> ep) {
  static_assert(NSTAGE >= 2 && NSTAGE <= 4 && (BK == 32 || BK == 64), "stages");
  constexpr int TT = kGemmBigT, NW = 4;
  constexpr int NI = gemm16_pipe_requests(TT, BK, NW);  // copy requests per thread, operand and step
  constexpr int OPB = TT * BK * 2;                      // bytes of an operand's step
  constexpr int OP = 2 * OPB;
  __shared__ __attribute__((aligned(1024))) char lds[gemm16_big_lds_bytes(BK, NSTAGE)];

  const int tiles = tiles_m * tiles_n;
  const int batch = blockIdx.x / tiles, tile = blockIdx.x % tiles;
  int tm, tn;
  gemm_tile_of_block(tile, tiles_m, tiles_n, tm, tn, true);
  const int m0 = tm * TT, n0 = tn * TT;
  const int steps = K / BK;
  A += batch * bsa;
  B += batch * bsb;
  const int64_t a_step = A_KC ? BK : BK * lda;
  const int64_t b_step = B_KC ? BK : BK * ldb;

  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int wm = (wave / 2) * 128;
  const int wn = (wave % 2) * 128;

  floatx16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const uint16_t* a16 = reinterpret_cast<const uint16_t*>(A);
  const uint16_t* b16 = reinterpret_cast<const uint16_t*>(B);
  int64_t src_a[NI], src_b[NI];
  gemm16_pipe_sources<A_KC, BK, TT, NW>(lda, m0, M, src_a);
  gemm16_pipe_sources<B_KC, BK, TT, NW>(ldb, n0, N, src_b);
  auto request = [&](int step, int copy) {
    gemm16_pipe_issue<NI, NW>(a16 + step * a_step, src_a, lds + copy * OP);
    gemm16_pipe_issue<NI, NW>(b16 + step * b_step, src_b, lds + copy * OP + OPB);
  };

  // The k loop is one stream of 16-deep slices.  While the sixteen MFMAs of a slice run, the
  // eight fragments of the next slice are read into the other half of `f` (the reads are dealt
  // out between the MFMAs with sched_group_barrier: left to itself the compiler reads each
  // fragment right before its use and waits for it).  Before the last slice of a step comes
  // the step's one synchronisation: the data of the next step has arrived (all but the
  // NSTAGE - 2 younger steps' copies), no wave reads the current step's tiles any more (their
  // last fragments are in registers), so the copy of step it + NSTAGE may overwrite them.
  constexpr int NS = BK / 16;
  constexpr int RA = A_KC ? 1 : 2, RB = B_KC ? 1 : 2;  // LDS reads per fragment
  uint4 f[2][8];
  auto read_frags = [&](int buf, int step, int ks) {  // B first: every MFMA group needs all four
    const char* la = lds + (step % NSTAGE) * OP;
    const char* lb = la + OPB;
#pragma unroll
    for (int i = 0; i < 4; ++i) f[buf][4 + i] = gemm16_pipe_frag<B_KC, BK, TT>(lb, wn + 32 * i, ks, lane);
#pragma unroll
    for (int i = 0; i < 4; ++i) f[buf][i] = gemm16_pipe_frag<A_KC, BK, TT>(la, wm + 32 * i, ks, lane);
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = GemmMma16<T>::run(f[buf][i], f[buf][4 + j], acc[i][j]);
  };
  // Slice ks of step `it`.  MODE 0: steady state (a copy is requested at the step's
  // synchronisation, the next step exists); 1: the product's last steps (nothing left to
  // request, every copy is waited for); 2: the very last slice (nothing left to read either).
  auto slice = [&](int it, int ks, auto mode) {
    constexpr int MODE = decltype(mode)::value;
    const int buf = ks % 2;
    if (ks == NS - 1) {
      if constexpr (MODE != 0 || NSTAGE == 2) MG_WAIT_VMCNT(0);
      else MG_WAIT_VMCNT(2 * NI * (NSTAGE - 2));
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if constexpr (MODE == 0) request(it + NSTAGE, it % NSTAGE);
      if constexpr (MODE != 2) read_frags(buf ^ 1, it + 1, 0);
    } else {
      read_frags(buf ^ 1, it, ks + 1);
    }
    multiply(buf);
    if constexpr (MODE != 2) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {  // four groups of (4 MFMAs, a quarter of the reads)
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, RA + RB, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  static_assert(NS % 2 == 0, "a step ends on the second fragment buffer");
#pragma unroll
  for (int s = 0; s < NSTAGE; ++s)
    if (s < steps) request(s, s);
  if (steps > NSTAGE - 1) MG_WAIT_VMCNT(2 * NI * (NSTAGE - 1));
  else MG_WAIT_VMCNT(0);
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  read_frags(0, 0, 0);
  // The loop body starts at a step's synchronisation (where nothing is outstanding anyway, so
  // what the compiler assumes at a loop head costs nothing) and runs on through the first
  // slices of the next step.
#pragma unroll
  for (int ks = 0; ks < NS - 1; ++ks) slice(0, ks, std::integral_constant<int, 0>{});
  int it = 0;
  for (; it < steps - NSTAGE; ++it) {
    slice(it, NS - 1, std::integral_constant<int, 0>{});
#pragma unroll
    for (int ks = 0; ks < NS - 1; ++ks) slice(it + 1, ks, std::integral_constant<int, 0>{});
  }
  for (; it < steps - 1; ++it) {
    slice(it, NS - 1, std::integral_constant<int, 1>{});
#pragma unroll
    for (int ks = 0; ks < NS - 1; ++ks) slice(it + 1, ks, std::integral_constant<int, 1>{});
  }
  slice(steps - 1, NS - 1, std::integral_constant<int, 2>{});
  __syncthreads();  // every wave is done with the staged tiles: their memory serves the output

  // The wave's 128 x 128 tile goes out as four 64 x 64 quadrants through its own strip of LDS.
  uint16_t* mine = reinterpret_cast<uint16_t*>(lds) + wave * 64 * kG16Stride;
#pragma unroll
  for (int qi = 0; qi < 2; ++qi)
#pragma unroll
    for (int qj = 0; qj < 2; ++qj) {
      floatx16 quad[2][2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) quad[i][j] = acc[2 * qi + i][2 * qj + j];
      gemm16_write_tile<T, HAS_BIAS, false>(quad, mine, bias, C, nullptr, M, N, ldc, bsc, batch, 0, 1, m0, n0,
                                            wm + 64 * qi, wn + 64 * qj, lane, ep);
      __syncthreads();  // the strip is read out before the next quadrant is written into it
    }
}

// Both products of a Linear layer's backward in one launch: workgroups [0, n_dw) take the
// K ranges of dW = dY^T X (their partial tiles are summed by linear_bwd_finish_kernel
// afterwards), the rest the tiles of dX = dY W.  The longer-running dW ranges start first
// and the dX tiles fill the CUs as those drain, where two launches each end in a tail of
// half-empty CUs (384 dX tiles on 256 CUs) and pay a launch apiece.  With
// dw.colsum_part set, the dW workgroups of the first tile column also produce the bias
// gradient's partial rows from the dY tiles they hold anyway.
template <typename T, int NSTAGE = 2, int TN = kGemmBN, int BK = 32>
__global__ __launch_bounds__(2 * TN, gemm16_pipe_occupancy(BK, NSTAGE, 128, TN)) void linear_bwd_16bit_kernel(
    Gemm16Problem<T> dw, Gemm16Problem<T> dx, int n_dw) {
  __shared__ __attribute__((aligned(1024))) char lds[gemm16_pipe_lds_bytes(BK, NSTAGE, 128, TN)];
  const int bid = blockIdx.x;
  if (bid < n_dw) gemm16_pipe_block<T, false, false, false, true, BK, NSTAGE, 128, TN>(lds, bid, dw);
  else gemm16_pipe_block<T, true, false, false, false, BK, NSTAGE, 128, TN>(lds, bid - n_dw, dx);
}

// The same launch with the dX tiles (128 x 384: whole rows of a 384-wide layer input) continuing
// as the backward of the LayerNorm that produced the layer's input (gemm16_ln_bwd_tile).
template <typename T>
__global__ __launch_bounds__(2 * kGemmWideBN, 1) void linear_bwd_ln_16bit_kernel(Gemm16Problem<T> dw, Gemm16Problem<T> dx,
                                                                                 int n_dw) {
  __shared__ __attribute__((aligned(1024))) char lds[gemm16_pipe_lds_bytes(64, 2, 128, kGemmWideBN)];
  const int bid = blockIdx.x;
  if (bid < n_dw) gemm16_pipe_block<T, false, false, false, true, 64, 2, 128, kGemmWideBN>(lds, bid, dw);
  else gemm16_pipe_block<T, true, false, false, false, 64, 2, 128, kGemmWideBN, true>(lds, bid - n_dw, dx);
}

// ------------------------------------------------------------------------------------
// fp32 product with the tiles copied global memory -> LDS by `global_load_lds_dwordx4`, two
// copies of each 128 x 32 tile: the copy of k-step i + 1 runs under the MFMAs of step i with
// one barrier per step and no registers or VALU work spent on staging.  Same tiles, same
// wave layout, same k order inside a step as gemm_f32_mfma_kernel (MFMA j of k-group g
// multiplies k in {g*8 + j, g*8 + 4 + j}), so the two kernels give identical bits.
// Requires K % 32 == 0 on top of that kernel's alignment conditions.
//
// LDS image of one operand's step (16 KB):
//   k-contiguous: [128 rows][8 chunks of 4 k], chunk c of row r at position c ^ (r/2 % 8)
//     (sixteen consecutive rows of a 128-bit fragment read hit sixteen bank groups);
//   otherwise: [32 k][32 chunks of 4 rows], chunk c of k-row kk at position
//     c ^ (8 * (kk/4 % 2)): the two halves of a wave read k and k + 4 of the same rows, 128
//     bytes apart in the banks.
// ------------------------------------------------------------------------------------

template <bool KC>
__device__ __forceinline__ void gemm32_pipe_sources(int64_t ld, int o0, int O, int64_t (&src)[4]) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int slot = (i * 4 + wave) * kWave + lane;  // 16-byte position in the LDS image
    if constexpr (KC) {
      const int r = slot / 8, c = (slot % 8) ^ ((r / 2) % 8);
      src[i] = static_cast<int64_t>(min(o0 + r, O - 1)) * ld + c * 4;  // rows past the edge are never stored
    } else {
      const int kk = slot / 32, c = (slot % 32) ^ (8 * ((kk / 4) % 2));
      const int o = o0 + c * 4;
      src[i] = static_cast<int64_t>(kk) * ld + (o < O ? o : o0);
    }
  }
}

// See gemm16_pipe_issue for why this is assembly.
__device__ __forceinline__ void gemm32_pipe_issue(const float* base, const int64_t* src, char* lds_step) {
  using lds_ptr = __attribute__((address_space(3))) char*;
  const int wave = threadIdx.x / kWave;
  const unsigned dst = static_cast<unsigned>(reinterpret_cast<uintptr_t>((lds_ptr)lds_step)) + wave * 1024;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const unsigned dst_i = __builtin_amdgcn_readfirstlane(dst + i * 4096);
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst_i), "v"(base + src[i]) : "memory");
  }
}

// MFMA operand values of one 32-wide tile for k-group g (see gemm_read_frag).
template <bool KC>
__device__ __forceinline__ void gemm32_pipe_frag(const char* __restrict__ lds_step, int o_base, int g, int lane,
                                                 float (&f)[4]) {
  const int o = o_base + lane % 32;
  if constexpr (KC) {
    const int c = g * 2 + lane / 32;
    const float4 r = *reinterpret_cast<const float4*>(lds_step + o * 128 + ((c ^ ((o / 2) % 8)) * 16));
    f[0] = r.x; f[1] = r.y; f[2] = r.z; f[3] = r.w;
  } else {
    const int kk = g * 8 + (lane / 32) * 4;  // (kk / 4) % 2 == lane / 32 for all four k of this lane
    const char* at = lds_step + kk * 512 + ((((o / 4) ^ (8 * (lane / 32))) * 16) + (o % 4) * 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) f[j] = *reinterpret_cast<const float*>(at + j * 512);
  }
}

// SPLIT_K: a work item is (K range, batch, tile); the fp32 partial tiles go to
// partial[(split * batches + batch), M, N] and gemm_splitk_reduce_kernel adds them up in a
// fixed order (for outputs with too few tiles to fill the device, e.g. a 10-class head).
template <bool A_KC, bool B_KC, bool HAS_BIAS, bool SPLIT_K>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_f32_pipe_kernel(
    const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ bias, float* __restrict__ C,
    float* __restrict__ partial, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int64_t bsa, int64_t bsb,
    int64_t bsc, int tiles_m, int tiles_n, int batches, int k_per_split, int total_work, GemmEpilogue<float> ep_in) {
  constexpr int OP = kGemmBM * kGemmBK * 4;  // bytes of one operand's step
  __shared__ __attribute__((aligned(1024))) char lds[2][2][OP];

  const int tiles = tiles_m * tiles_n;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int wm = (wave / 2) * 64;
  const int wn = (wave % 2) * 64;
  const int64_t a_step = A_KC ? kGemmBK : kGemmBK * lda;
  const int64_t b_step = B_KC ? kGemmBK : kGemmBK * ldb;
  // The grid holds at most the workgroups that are resident at once; each takes output tiles
  // work, work + gridDim.x, ... (see gemm_f32_mfma_kernel).
  for (int work = blockIdx.x; work < total_work; work += gridDim.x) {
    const int split = SPLIT_K ? work / (tiles * batches) : 0;
    const int in_split = SPLIT_K ? work % (tiles * batches) : work;
    const int batch = in_split / tiles;
    int tm, tn;
    gemm_tile_of_block(in_split % tiles, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * kGemmBM;
    const int n0 = tn * kGemmBN;
    const int k_begin = SPLIT_K ? split * k_per_split : 0;
    const int steps = (SPLIT_K ? min(K - k_begin, k_per_split) : K) / kGemmBK;
    const float* a = A + batch * bsa + (A_KC ? static_cast<int64_t>(k_begin) : k_begin * lda);
    const float* b = B + batch * bsb + (B_KC ? static_cast<int64_t>(k_begin) : k_begin * ldb);
    float* c = C + batch * bsc;
    GemmEpilogue<float> ep = ep_in;
    if (ep.residual) ep.residual += batch * bsc;
    if (ep.relu_mask) ep.relu_mask += batch * bsc;

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    int64_t src_a[4], src_b[4];
    gemm32_pipe_sources<A_KC>(lda, m0, M, src_a);
    gemm32_pipe_sources<B_KC>(ldb, n0, N, src_b);
    gemm32_pipe_issue(a, src_a, lds[0][0]);
    gemm32_pipe_issue(b, src_b, lds[0][1]);
    for (int it = 0; it < steps; ++it) {
      const int cur = it & 1;
      // This wave's copies of step `it` have landed; the barrier covers the other waves' and
      // tells that everyone is done reading the other copy.  (A plain barrier: __syncthreads()
      // would be the same here, every copy being waited for, but costs a fence.)
      MG_WAIT_VMCNT(0);
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if (it + 1 < steps) {
        gemm32_pipe_issue(a + (it + 1) * a_step, src_a, lds[cur ^ 1][0]);
        gemm32_pipe_issue(b + (it + 1) * b_step, src_b, lds[cur ^ 1][1]);
      }
      const char* la = lds[cur][0];
      const char* lb = lds[cur][1];
      // The fragments of k-group g + 1 are requested before the products of group g.
      float fa[2][2][4], fb[2][2][4];
      gemm32_pipe_frag<A_KC>(la, wm, 0, lane, fa[0][0]);
      gemm32_pipe_frag<A_KC>(la, wm + 32, 0, lane, fa[0][1]);
      gemm32_pipe_frag<B_KC>(lb, wn, 0, lane, fb[0][0]);
      gemm32_pipe_frag<B_KC>(lb, wn + 32, 0, lane, fb[0][1]);
#pragma unroll
      for (int g = 0; g < kGemmBK / 8; ++g) {
        const int p = g % 2, n = p ^ 1;
        if (g + 1 < kGemmBK / 8) {
          gemm32_pipe_frag<A_KC>(la, wm, g + 1, lane, fa[n][0]);
          gemm32_pipe_frag<A_KC>(la, wm + 32, g + 1, lane, fa[n][1]);
          gemm32_pipe_frag<B_KC>(lb, wn, g + 1, lane, fb[n][0]);
          gemm32_pipe_frag<B_KC>(lb, wn + 32, g + 1, lane, fb[n][1]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int tj = 0; tj < 2; ++tj)
              acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[p][ti][j], fb[p][tj][j], acc[ti][tj], 0, 0, 0);
      }
    }
    // The next tile's first copy goes into lds[0]: every wave must be done reading it.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // Accumulator element r of a lane is row (r/4)*8 + (lane/32)*4 + r%4, column lane%32.
#pragma unroll
    for (int ti = 0; ti < 2; ++ti)
#pragma unroll
      for (int tj = 0; tj < 2; ++tj) {
        const int col = n0 + wn + tj * 32 + lane % 32;
        if (col >= N) continue;
        const float bv = (HAS_BIAS && !SPLIT_K) ? bias[col] : 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = m0 + wm + ti * 32 + (r / 4) * 8 + (lane / 32) * 4 + (r % 4);
          if (row < M) {
            if constexpr (SPLIT_K) {
              partial[((static_cast<int64_t>(split) * batches + batch) * M + row) * N + col] = acc[ti][tj][r];
            } else {
              const int64_t at = static_cast<int64_t>(row) * ldc + col;
              c[at] = gemm_finish<float>(acc[ti][tj][r] + bv, ep, at);
            }
          }
        }
      }
  }  // tiles of this workgroup
}

// out[i] = sum_s partial[s * slice + i] (+ bias[i % N]) for i < numel <= slice, converted to T.  One thread
// sums group g, four consecutive outputs, over all K ranges: range s goes to one of eight
// running sums, number (s / 4 % 2, s % 4), in increasing s, and the eight meet as
// ((a00 + a10) + (a01 + a11)) + ((a02 + a12) + (a03 + a13)).  The order is fixed, so the result is
// deterministic; it is the order of an earlier form of this reduction (four waves summing
// every fourth range each and meeting in LDS), kept so that results did not change, with
// eight independent 16-byte loads in flight per thread and no barrier.
// TILED: the partials are whole 128 x 128 tiles in accumulator order (kG16PartialTile), numel
// = slice = their count per K range, and a group of four is four consecutive rows of one
// column of `out` (rows x N per batch; tiles_n tile columns; rows and columns past the matrix
// are dropped).
template <typename T, bool HAS_BIAS, bool TILED = false, bool STREAM = false>
__device__ __forceinline__ void gemm_splitk_reduce_group(int64_t g, const float* __restrict__ partial,
                                                         const T* __restrict__ bias, T* __restrict__ out, int64_t numel,
                                                         int64_t slice, int splits, int N, const GemmEpilogue<T>& ep,
                                                         int rows = 0, int tiles_n = 0) {
  const int64_t i = g * 4;
  if (i >= numel) return;
  float r[4];
  if (TILED || i + 3 < numel) {
    float4 acc[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[h][j] = make_float4(0.f, 0.f, 0.f, 0.f);
    const float* p = partial + i;
    constexpr int NB = 8;  // K ranges in flight per thread (2 or 1 measured 2-7 % slower on a step's sums)
    for (int s0 = 0; s0 < splits; s0 += 8) {
#pragma unroll
      for (int h = 0; h < 8; h += NB) {
        float4 v[NB];
#pragma unroll
        for (int e = 0; e < NB; ++e)
          if (s0 + h + e >= splits) {
            v[e] = make_float4(0.f, 0.f, 0.f, 0.f);
          } else if constexpr (STREAM) {
            // read once, long after it was written: a streaming load that leaves the caches to
            // the tensors of the next step (a step's deferred sums: 137 -> 103 us)
            const floatx4 nt =
                __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(p + static_cast<int64_t>(s0 + h + e) * slice));
            v[e] = make_float4(nt[0], nt[1], nt[2], nt[3]);
          } else {
            v[e] = *reinterpret_cast<const float4*>(p + static_cast<int64_t>(s0 + h + e) * slice);
          }
#pragma unroll
        for (int e = 0; e < NB; ++e) {
          if (s0 + h + e < splits) {  // (adding the zero would turn a -0 sum into +0)
            float4& a = acc[(h + e) / 4][(h + e) % 4];
            a.x += v[e].x; a.y += v[e].y; a.z += v[e].z; a.w += v[e].w;
          }
        }
      }
    }
    float4 t[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      t[j] = make_float4(acc[0][j].x + acc[1][j].x, acc[0][j].y + acc[1][j].y, acc[0][j].z + acc[1][j].z,
                         acc[0][j].w + acc[1][j].w);
    r[0] = (t[0].x + t[1].x) + (t[2].x + t[3].x);
    r[1] = (t[0].y + t[1].y) + (t[2].y + t[3].y);
    r[2] = (t[0].z + t[1].z) + (t[2].z + t[3].z);
    r[3] = (t[0].w + t[1].w) + (t[2].w + t[3].w);
  } else {
    // the last, partial group of an untiled slice: element by element, four running sums
    float a[4][3];
#pragma unroll
    for (int j = 0; j < 4; ++j) a[j][0] = a[j][1] = a[j][2] = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float* p = partial + static_cast<int64_t>(s) * slice + i;
      a[s % 4][0] += p[0];
      if (i + 1 < numel) a[s % 4][1] += p[1];
      if (i + 2 < numel) a[s % 4][2] += p[2];
    }
#pragma unroll
    for (int e = 0; e < 3; ++e) r[e] = ((a[0][e] + 0.f) + (a[1][e] + 0.f)) + ((a[2][e] + 0.f) + (a[3][e] + 0.f));
    r[3] = 0.f;
  }
  if constexpr (TILED) {
    // g = ((((t * 4 + wave) * 2 + ti) * 2 + tj) * 4 + q) * 64 + lane
    const int lane = static_cast<int>(g % 64), q = static_cast<int>(g / 64 % 4), tj = static_cast<int>(g / 256 % 2),
              ti = static_cast<int>(g / 512 % 2), wave = static_cast<int>(g / 1024 % 4);
    const int64_t t = g / 4096;  // tile over (batch, tile row, tile column)
    const int tiles_m = (rows + kGemmBM - 1) / kGemmBM;
    const int tn = static_cast<int>(t % tiles_n), tm = static_cast<int>(t / tiles_n % tiles_m);
    const int64_t batch = t / tiles_n / tiles_m;
    const int row = tm * kGemmBM + (wave / 2) * 64 + ti * 32 + q * 8 + (lane / 32) * 4;
    const int col = tn * kGemmBN + (wave % 2) * 64 + tj * 32 + lane % 32;
    if (col >= N) return;
    const float bv = HAS_BIAS ? to_float(bias[col]) : 0.f;
    for (int e = 0; e < 4 && row + e < rows; ++e) {
      const int64_t at = (batch * rows + row + e) * N + col;
      out[at] = gemm_finish<T>(r[e] + bv, ep, at);
    }
  } else {
    for (int e = 0; e < 4 && i + e < numel; ++e) {
      const float bv = HAS_BIAS ? to_float(bias[(i + e) % N]) : 0.f;
      out[i + e] = gemm_finish<T>(r[e] + bv, ep, i + e);
    }
  }
}

template <typename T, bool HAS_BIAS, bool TILED = false>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ partial,
                                                                 const T* __restrict__ bias, T* __restrict__ out,
                                                                 int64_t numel, int64_t slice, int splits, int N,
                                                                 GemmEpilogue<T> ep, int rows = 0, int tiles_n = 0) {
  gemm_splitk_reduce_group<T, HAS_BIAS, TILED>(static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x, partial, bias, out,
                                               numel, slice, splits, N, ep, rows, tiles_n);
}

// db[c] = sum over the `groups` partial rows db_part[g][c], 64 columns per 256 threads (`tid`
// of them, column block `bx`): every fourth row per 64 threads, then (t0 + t1) + (t2 + t3).
// `sums_` is 256 floats of LDS; every one of the 256 threads must make the call.
template <typename T>
__device__ __forceinline__ void linear_bwd_db_block(float* __restrict__ sums_, int tid, int bx,
                                                    const float* __restrict__ db_part, T* __restrict__ db, int groups,
                                                    int N) {
  float(&sums)[4][64] = *reinterpret_cast<float(*)[4][64]>(sums_);
  const int cx = tid % 64, sl = tid / 64;
  const int c = bx * 64 + cx;
  float a0 = 0.f, a1 = 0.f;
  if (c < N) {
    int g = sl;
    for (; g + 4 < groups; g += 8) {
      a0 += db_part[static_cast<int64_t>(g) * N + c];
      a1 += db_part[static_cast<int64_t>(g + 4) * N + c];
    }
    for (; g < groups; g += 4) a0 += db_part[static_cast<int64_t>(g) * N + c];
  }
  sums[sl][cx] = a0 + a1;
  __syncthreads();
  if (sl == 0 && c < N) db[c] = from_float<T>((sums[0][cx] + sums[1][cx]) + (sums[2][cx] + sums[3][cx]));
}

// What follows the common launch of a Linear layer's backward: workgroups [0, dw_blocks) sum
// the K ranges of dW (gemm_splitk_reduce_block), the rest sum the `groups` partial rows of
// the bias gradient that the launch left (one per K range), 64 columns per workgroup,
// every fourth row per 64 threads, then (t0 + t1) + (t2 + t3).  Fixed order, no atomics.
// dw_blocks = ceil(slice / 1024): a thread sums four consecutive values of a partial tile.
template <typename T>
__global__ __launch_bounds__(256) void linear_bwd_finish_kernel(const float* __restrict__ partial, T* __restrict__ dw,
                                                                int dw_rows, int64_t slice, int splits, int K,
                                                                int dw_blocks, const float* __restrict__ db_part,
                                                                T* __restrict__ db, int groups, int N) {
  __shared__ float sums[256];
  const int bid = blockIdx.x;
  if (bid < dw_blocks) {
    // dW is (dw_rows, K); the partial tiles cover the (N, K) product of the launch
    gemm_splitk_reduce_group<T, false, true>(static_cast<int64_t>(bid) * 256 + threadIdx.x, partial,
                                             static_cast<const T*>(nullptr), dw, slice, slice, splits, K,
                                             GemmEpilogue<T>{nullptr, nullptr, 0}, dw_rows, (K + kGemmBN - 1) / kGemmBN);
    return;
  }
  linear_bwd_db_block<T>(sums, threadIdx.x, bid - dw_blocks, db_part, db, groups, N);
}

}  // namespace mg
