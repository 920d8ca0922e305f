// Axis sums (the bias gradient db = sum over rows of dY) and relu_grad.
#include "mg_device.h"
#include "mg_internal.h"
#include "mg_rows.h"

namespace mg {

// Stage 1 of dst(o, i) = sum_r a(o, r, i): a workgroup is TX column threads by 256 / TX row
// lanes; a thread sums every (256 / TX)-th row of its slab for VEC columns with 16-byte
// loads (narrow matrices get more row lanes instead of idle column threads).  DIRECT writes
// the final value (one slab, one row lane); otherwise fp32 partials
// (outer, slab * row_lanes + lane, inner) go to scratch and reduce_partials_cw_kernel finishes
// in a fixed order.  No atomics.
template <typename T, int VEC, bool DIRECT>
__global__ __launch_bounds__(256) void colsum_partial_kernel(const T* __restrict__ a, float* __restrict__ part,
                                                             T* __restrict__ dst, int64_t reduce, int64_t inner,
                                                             int64_t rows_per_chunk, int tx_log2) {
  const int tx = 1 << tx_log2;
  const int ry = 256 >> tx_log2;
  const int cx = threadIdx.x & (tx - 1);
  const int ly = threadIdx.x >> tx_log2;
  const int64_t col = (static_cast<int64_t>(blockIdx.x) * tx + cx) * VEC;
  if (col >= inner) return;
  const int64_t chunk = blockIdx.y;
  const int64_t o = blockIdx.z;
  const int64_t r0 = chunk * rows_per_chunk + ly;
  const int64_t r1 = min(chunk * rows_per_chunk + rows_per_chunk, reduce);
  const T* base = a + (o * reduce) * inner + col;
  const int64_t step = static_cast<int64_t>(ry) * inner;  // elements between this thread's rows
  float acc[4][VEC];
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[u][e] = 0.f;
  int64_t r = r0;
  const T* p = base + r0 * inner;
  for (; r + 3 * ry < r1; r += 4 * ry, p += 4 * step) {
    float v[4][VEC];
#pragma unroll
    for (int u = 0; u < 4; ++u) VecIO<T, VEC>::load(p + u * step, v[u]);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[u][e] += v[u][e];
  }
  for (; r < r1; r += ry, p += step) {
    float v[VEC];
    VecIO<T, VEC>::load(p, v);
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[0][e] += v[e];
  }
  float out[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) out[e] = (acc[0][e] + acc[1][e]) + (acc[2][e] + acc[3][e]);
  if constexpr (DIRECT) {
    VecIO<T, VEC>::store(dst + o * inner + col, out);
  } else {
    float* q = part + ((o * gridDim.y + chunk) * ry + ly) * inner + col;
#pragma unroll
    for (int e = 0; e < VEC; ++e) q[e] = out[e];
  }
}

// One-launch form for wide matrices: a 1024-thread workgroup owns a 128-byte-wide slab of
// columns (eight 16-byte pieces) for every row, 128 row lanes deep, so a wave's load reads
// eight whole 128-byte lines and nothing a workgroup fetches is shared with another.  Each
// thread sums every 128th row with eight loads in flight; the 128 row lanes are then added
// through LDS in a fixed order and the result is stored directly: no partial sums in
// memory, no second launch, no atomics.
template <typename T, int VEC>
__global__ __launch_bounds__(1024) void colsum_slab_kernel(const T* __restrict__ a, T* __restrict__ dst,
                                                           int64_t reduce, int64_t inner) {
  constexpr int PIECES = 8;             // 16-byte pieces per slab row
  constexpr int LANES = 1024 / PIECES;  // row lanes
  constexpr int NCOL = PIECES * VEC;    // columns of a slab
  constexpr int SL = 1024 / NCOL;       // row-lane groups in the first LDS pass
  __shared__ float tile[LANES][NCOL + 1];
  __shared__ float tile2[SL][NCOL + 1];
  const int cx = threadIdx.x % PIECES;
  const int ly = threadIdx.x / PIECES;
  const int64_t col = (static_cast<int64_t>(blockIdx.x) * PIECES + cx) * VEC;
  const int64_t o = blockIdx.y;
  float acc[4][VEC];
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[u][e] = 0.f;
  if (col < inner) {
    const int64_t step = static_cast<int64_t>(LANES) * inner;
    const T* p = a + (o * reduce + ly) * inner + col;
    int64_t r = ly;
    for (; r + 7 * LANES < reduce; r += 8 * LANES, p += 8 * step) {
      float v[8][VEC];
#pragma unroll
      for (int u = 0; u < 8; ++u) VecIO<T, VEC>::load(p + u * step, v[u]);
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[u & 3][e] += v[u][e];
    }
    for (; r < reduce; r += LANES, p += step) {
      float v[VEC];
      VecIO<T, VEC>::load(p, v);
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[0][e] += v[e];
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) tile[ly][cx * VEC + e] = (acc[0][e] + acc[1][e]) + (acc[2][e] + acc[3][e]);
  __syncthreads();
  {
    const int c = threadIdx.x % NCOL, s = threadIdx.x / NCOL;
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < LANES / SL; ++k) t += tile[s * (LANES / SL) + k][c];
    tile2[s][c] = t;
  }
  __syncthreads();
  if (threadIdx.x < NCOL) {
    const int64_t c = static_cast<int64_t>(blockIdx.x) * NCOL + threadIdx.x;
    float t = 0.f;
#pragma unroll
    for (int s = 0; s < SL; ++s) t += tile2[s][threadIdx.x];
    if (c < inner) dst[o * inner + c] = from_float<T>(t);
  }
}

// Sum over the last axis (inner == 1): one wave per output element.
template <typename T>
__global__ __launch_bounds__(256) void rowsum_kernel(const T* __restrict__ a, T* __restrict__ dst, int64_t outer,
                                                     int64_t reduce) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (row >= outer) return;  // wave-uniform
  const int lane = threadIdx.x % kWave;
  float acc = 0.f;
  for (int64_t c = lane; c < reduce; c += kWave) acc += to_float(a[row * reduce + c]);
  acc = wave_sum(acc);
  if (lane == 0) dst[row] = from_float<T>(acc);
}

template <typename T>
__global__ __launch_bounds__(256) void relu_grad_kernel(const T* __restrict__ out, const T* __restrict__ up,
                                                        T* __restrict__ dst, int64_t n) {
  constexpr int VEC = WideVec<T>::value;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * VEC;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * VEC; i < n; i += stride) {
    if (i + VEC <= n) {
      float o[VEC], u[VEC], r[VEC];
      VecIO<T, VEC>::load(out + i, o);
      VecIO<T, VEC>::load(up + i, u);
#pragma unroll
      for (int e = 0; e < VEC; ++e) r[e] = o[e] > 0.f ? u[e] : 0.f;
      VecIO<T, VEC>::store(dst + i, r);
    } else {
      for (int64_t j = i; j < n; ++j) dst[j] = to_float(out[j]) > 0.f ? up[j] : from_float<T>(0.f);
    }
  }
}

template <typename T>
static int colsum_typed(const T* a, T* dst, int64_t outer, int64_t reduce, int64_t inner, hipStream_t stream) {
  if (reduce == 0) {
    // zero fill by kernel, not hipMemsetAsync: safe to record into a HIP graph
    const int dtype = sizeof(T) == 4 ? MG_F32 : MG_F16;  // all-zero bits are zero in every float type
    return mg_fill(dst, 0.0, outer * inner, dtype, stream);
  }
  if (inner == 1) {
    hipLaunchKernelGGL((rowsum_kernel<T>), dim3(static_cast<unsigned>(ceil_div(outer, 4))), dim3(256), 0, stream, a, dst,
                       outer, reduce);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }
  constexpr int WIDE = WideVec<T>::value;
  const bool wide = inner % WIDE == 0 && aligned16(a) && aligned16(dst);
  const int vec = wide ? WIDE : 1;
  // Wide matrices take the one-launch kernel: always when there is a 128-byte column slab
  // for every CU; with slabs for half the CUs only up to 48 MiB of input (half the CUs
  // stream about 4 TB/s against 5 for the two-stage form on all of them, which outweighs
  // the saved launch beyond roughly 40 MB).
  const int64_t slabs = ceil_div(inner, 8 * WIDE) * outer;
  const int64_t cus = device_info().cu_count;
  const bool slab_fits = slabs >= cus || (2 * slabs >= cus && outer * reduce * inner * static_cast<int64_t>(sizeof(T)) <=
                                                                   (int64_t{48} << 20));
  if (wide && outer <= 65535 && reduce >= 128 && slab_fits && env_int("MOGRAD_HIP_COLSUM_SLAB", 1) != 0) {
    hipLaunchKernelGGL((colsum_slab_kernel<T, WIDE>),
                       dim3(static_cast<unsigned>(ceil_div(inner, 8 * WIDE)), static_cast<unsigned>(outer)), dim3(1024),
                       0, stream, a, dst, reduce, inner);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }
  // Column threads per workgroup: the smallest power of two covering the columns, at most 256.
  int tx_log2 = 3;
  while (tx_log2 < 8 && (int64_t{1} << tx_log2) * vec < inner) ++tx_log2;
  const int tx = 1 << tx_log2, ry = 256 >> tx_log2;
  const int64_t col_blocks = ceil_div(inner, static_cast<int64_t>(tx) * vec);
  if (outer > 65535) return fail(MG_ERR_UNSUPPORTED, "sum_axis: outer=%lld exceeds 65535", static_cast<long long>(outer));
  // Enough slabs to fill the device, each at least 32 rows per row lane (fewer, longer
  // slabs keep the fp32 partial sums a small fraction of the traffic).
  int64_t chunks = ceil_div(static_cast<int64_t>(device_info().cu_count) * env_int("MOGRAD_HIP_COLSUM_WG_PER_CU", 4),
                            col_blocks * outer);
  const int64_t max_chunks = ceil_div(reduce, static_cast<int64_t>(env_int("MOGRAD_HIP_COLSUM_MIN_ROWS", 32)) * ry);
  if (chunks > max_chunks) chunks = max_chunks;
  if (chunks < 1) chunks = 1;
  if (chunks > 65535) chunks = 65535;
  const int64_t rows_per_chunk = ceil_div(reduce, chunks);
  chunks = ceil_div(reduce, rows_per_chunk);
  const dim3 grid(static_cast<unsigned>(col_blocks), static_cast<unsigned>(chunks), static_cast<unsigned>(outer));
  if (chunks == 1 && ry == 1) {
    if (wide)
      hipLaunchKernelGGL((colsum_partial_kernel<T, WIDE, true>), grid, dim3(256), 0, stream, a, nullptr, dst, reduce,
                         inner, rows_per_chunk, tx_log2);
    else
      hipLaunchKernelGGL((colsum_partial_kernel<T, 1, true>), grid, dim3(256), 0, stream, a, nullptr, dst, reduce, inner,
                         rows_per_chunk, tx_log2);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }
  const int64_t groups = chunks * ry;
  Scratch part;
  MG_TRY(part.take(outer * groups * inner * static_cast<int64_t>(sizeof(float))));
  if (wide)
    hipLaunchKernelGGL((colsum_partial_kernel<T, WIDE, false>), grid, dim3(256), 0, stream, a, part.as<float>(), dst,
                       reduce, inner, rows_per_chunk, tx_log2);
  else
    hipLaunchKernelGGL((colsum_partial_kernel<T, 1, false>), grid, dim3(256), 0, stream, a, part.as<float>(), dst,
                       reduce, inner, rows_per_chunk, tx_log2);
  MG_LAUNCH_CHECK();
  for (int64_t o = 0; o < outer; ++o) {
    launch_reduce_partials<T>(part.as<float>() + o * groups * inner, dst + o * inner, nullptr, nullptr, groups, inner,
                              device_info().cu_count, stream);
    MG_LAUNCH_CHECK();
  }
  return MG_OK;
}

int colsum_dispatch(const void* a, void* dst, int64_t outer, int64_t reduce, int64_t inner, int dtype,
                    hipStream_t stream) {
  if (!is_float_dtype(dtype)) return fail(MG_ERR_INVALID, "sum_axis: unsupported dtype %s", dtype_name(dtype));
  if (outer < 0 || reduce < 0 || inner < 0)
    return fail(MG_ERR_INVALID, "sum_axis: bad shape (%lld, %lld, %lld)", static_cast<long long>(outer),
                static_cast<long long>(reduce), static_cast<long long>(inner));
  if (outer == 0 || inner == 0) return MG_OK;
  if (!dst || (reduce > 0 && !a)) return fail(MG_ERR_INVALID, "sum_axis: null pointer argument");
  switch (dtype) {
    case MG_F32: return colsum_typed(static_cast<const float*>(a), static_cast<float*>(dst), outer, reduce, inner, stream);
    case MG_F16: return colsum_typed(static_cast<const f16_t*>(a), static_cast<f16_t*>(dst), outer, reduce, inner, stream);
    default: return colsum_typed(static_cast<const bf16_t*>(a), static_cast<bf16_t*>(dst), outer, reduce, inner, stream);
  }
}

template <typename T>
static int relu_grad_typed(const void* out, const void* up, void* dst, int64_t n, hipStream_t stream) {
  constexpr int VEC = WideVec<T>::value;
  if (!aligned16(out) || !aligned16(up) || !aligned16(dst))
    return fail(MG_ERR_INVALID, "relu_grad: pointers must be 16-byte aligned");
  int64_t blocks = ceil_div(n, 256 * VEC);
  const int64_t cap = static_cast<int64_t>(device_info().cu_count) * 16;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL((relu_grad_kernel<T>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                     static_cast<const T*>(out), static_cast<const T*>(up), static_cast<T*>(dst), n);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

}  // namespace mg

extern "C" {

int mg_sum_axis(const void* a, void* dst, int64_t outer, int64_t reduce, int64_t inner, int dtype, mg_stream stream) {
  return mg::colsum_dispatch(a, dst, outer, reduce, inner, dtype, mg::to_stream(stream));
}

int mg_relu_grad(const void* out, const void* upstream, void* dst, int64_t n, int dtype, mg_stream stream) {
  if (!mg::is_float_dtype(dtype)) return mg::fail(MG_ERR_INVALID, "relu_grad: unsupported dtype %s", mg::dtype_name(dtype));
  if (n < 0) return mg::fail(MG_ERR_INVALID, "relu_grad: negative size");
  if (n == 0) return MG_OK;
  if (!out || !upstream || !dst) return mg::fail(MG_ERR_INVALID, "relu_grad: null pointer argument");
  hipStream_t s = mg::to_stream(stream);
  switch (dtype) {
    case MG_F32: return mg::relu_grad_typed<float>(out, upstream, dst, n, s);
    case MG_F16: return mg::relu_grad_typed<mg::f16_t>(out, upstream, dst, n, s);
    default: return mg::relu_grad_typed<mg::bf16_t>(out, upstream, dst, n, s);
  }
}

}  // extern "C"
