// Row softmax, its gradient, and argmax along an axis: the unfused attention fallback and
// the accuracy metric of the reference's training loops.  One wave per row, 16-byte
// accesses, DPP wave reductions, fp32 arithmetic.
#include "mg_device.h"
#include "mg_internal.h"

namespace mg {

constexpr float kLog2e = 1.4426950408889634f;

// y = exp(x - max) / sum exp(x - max).  Pass 1: running maximum and rescaled sum in one
// sweep; pass 2 re-reads the row (it is still in cache) and writes the result.
// One wave, one row.  `xs`: elements between neighbours of the input row (1 whenever VEC > 1).
template <typename T, int VEC>
__device__ __forceinline__ void softmax_row(const T* __restrict__ xr, int64_t xs, T* __restrict__ yr, int64_t cols,
                                            int lane) {
  float m = -INFINITY, l = 0.f;
  for (int64_t c = static_cast<int64_t>(lane) * VEC; c < cols; c += kWave * VEC) {
    float v[VEC];
    VecIO<T, VEC>::load(xr + c * xs, v);
    float cm = v[0];
#pragma unroll
    for (int e = 1; e < VEC; ++e) cm = fmaxf(cm, v[e]);
    const float nm = fmaxf(m, cm);
    if (nm > -INFINITY) {
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < VEC; ++e) s += __builtin_amdgcn_exp2f((v[e] - nm) * kLog2e);
      l = l * __builtin_amdgcn_exp2f((m - nm) * kLog2e) + s;
      m = nm;
    }
  }
  const float gm = wave_max(m);
  l = (m > -INFINITY) ? l * __builtin_amdgcn_exp2f((m - gm) * kLog2e) : 0.f;
  const float inv = 1.0f / wave_sum(l);
  for (int64_t c = static_cast<int64_t>(lane) * VEC; c < cols; c += kWave * VEC) {
    float v[VEC];
    VecIO<T, VEC>::load(xr + c * xs, v);
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = __builtin_amdgcn_exp2f((v[e] - gm) * kLog2e) * inv;
    VecIO<T, VEC>::store(yr + c, v);
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void softmax_rows_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows,
                                                           int64_t cols) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (row >= rows) return;  // wave-uniform
  softmax_row<T, VEC>(x + row * cols, 1, y + row * cols, cols, threadIdx.x % kWave);
}

// The rows of a strided view: `v` holds the extents and strides of the dims in front of the
// last one, `xs` the stride of the last.  The result is row-major.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void softmax_view_kernel(const T* __restrict__ x, T* __restrict__ y, StridedView v,
                                                           int64_t xs, int64_t rows, int64_t cols) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (row >= rows) return;  // wave-uniform
  int64_t rem = row, off = 0;
  for (int d = v.rank - 1; d >= 0; --d) {
    const int64_t q = rem / v.shape[d];
    off += (rem - q * v.shape[d]) * v.stride[d];
    rem = q;
  }
  softmax_row<T, VEC>(x + off, xs, y + row * cols, cols, threadIdx.x % kWave);
}

// dst = y * (upstream - sum_c y * upstream)
template <typename T, int VEC>
__global__ __launch_bounds__(256) void softmax_grad_rows_kernel(const T* __restrict__ y, const T* __restrict__ up,
                                                                T* __restrict__ dst, int64_t rows, int64_t cols) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (row >= rows) return;
  const int lane = threadIdx.x % kWave;
  const T* yr = y + row * cols;
  const T* ur = up + row * cols;
  T* dr = dst + row * cols;
  float dot = 0.f;
  for (int64_t c = static_cast<int64_t>(lane) * VEC; c < cols; c += kWave * VEC) {
    float a[VEC], b[VEC];
    VecIO<T, VEC>::load(yr + c, a);
    VecIO<T, VEC>::load(ur + c, b);
#pragma unroll
    for (int e = 0; e < VEC; ++e) dot = fmaf(a[e], b[e], dot);
  }
  dot = wave_sum(dot);
  for (int64_t c = static_cast<int64_t>(lane) * VEC; c < cols; c += kWave * VEC) {
    float a[VEC], b[VEC];
    VecIO<T, VEC>::load(yr + c, a);
    VecIO<T, VEC>::load(ur + c, b);
#pragma unroll
    for (int e = 0; e < VEC; ++e) a[e] = a[e] * (b[e] - dot);
    VecIO<T, VEC>::store(dr + c, a);
  }
}

// First index of the largest value along the middle axis of (outer, reduce, inner), stored
// as a value of T.  A value replaces the best so far only if it is strictly greater, so
// ties go to the lowest index and NaN never wins; the search starts from -inf at index 0.
template <typename T>
__global__ __launch_bounds__(256) void argmax_last_kernel(const T* __restrict__ a, T* __restrict__ dst, int64_t outer,
                                                          int64_t reduce) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (row >= outer) return;
  const int lane = threadIdx.x % kWave;
  float best = -INFINITY;
  int64_t idx = 0;
  for (int64_t c = lane; c < reduce; c += kWave) {
    const float v = to_float(a[row * reduce + c]);
    if (v > best) {
      best = v;
      idx = c;
    }
  }
  // combine lanes: larger value wins, equal values go to the lower index
#pragma unroll
  for (int w = 1; w < kWave; w *= 2) {
    const float ob = __shfl_xor(best, w);
    const int64_t oi = __shfl_xor(static_cast<long long>(idx), w);
    if (ob > best || (ob == best && oi < idx)) {
      best = ob;
      idx = oi;
    }
  }
  if (lane == 0) dst[row] = from_float<T>(best > -INFINITY ? static_cast<float>(idx) : 0.f);
}

template <typename T>
__global__ __launch_bounds__(256) void argmax_mid_kernel(const T* __restrict__ a, T* __restrict__ dst, int64_t outer,
                                                         int64_t reduce, int64_t inner) {
  const int64_t flat = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (flat >= outer * inner) return;
  const int64_t o = flat / inner, i = flat % inner;
  float best = -INFINITY;
  int64_t idx = 0;
  for (int64_t r = 0; r < reduce; ++r) {
    const float v = to_float(a[(o * reduce + r) * inner + i]);
    if (v > best) {
      best = v;
      idx = r;
    }
  }
  dst[flat] = from_float<T>(static_cast<float>(idx));
}

template <typename T>
static int softmax_typed(const void* x, void* y, int64_t rows, int64_t cols, hipStream_t s) {
  constexpr int WIDE = WideVec<T>::value;
  const dim3 grid(static_cast<unsigned>(ceil_div(rows, 4)));
  if (cols % WIDE == 0 && aligned16(x) && aligned16(y))
    hipLaunchKernelGGL((softmax_rows_kernel<T, WIDE>), grid, dim3(256), 0, s, static_cast<const T*>(x),
                       static_cast<T*>(y), rows, cols);
  else
    hipLaunchKernelGGL((softmax_rows_kernel<T, 1>), grid, dim3(256), 0, s, static_cast<const T*>(x), static_cast<T*>(y),
                       rows, cols);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T>
static int softmax_view_typed(const void* x, void* y, const StridedView& v, int64_t xs, int64_t rows, int64_t cols,
                              bool wide, hipStream_t s) {
  constexpr int WIDE = WideVec<T>::value;
  const dim3 grid(static_cast<unsigned>(ceil_div(rows, 4)));
  if (wide && cols % WIDE == 0)
    hipLaunchKernelGGL((softmax_view_kernel<T, WIDE>), grid, dim3(256), 0, s, static_cast<const T*>(x), static_cast<T*>(y),
                       v, xs, rows, cols);
  else
    hipLaunchKernelGGL((softmax_view_kernel<T, 1>), grid, dim3(256), 0, s, static_cast<const T*>(x), static_cast<T*>(y), v,
                       xs, rows, cols);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T>
static int softmax_grad_typed(const void* y, const void* up, void* dst, int64_t rows, int64_t cols, hipStream_t s) {
  constexpr int WIDE = WideVec<T>::value;
  const dim3 grid(static_cast<unsigned>(ceil_div(rows, 4)));
  if (cols % WIDE == 0 && aligned16(y) && aligned16(up) && aligned16(dst))
    hipLaunchKernelGGL((softmax_grad_rows_kernel<T, WIDE>), grid, dim3(256), 0, s, static_cast<const T*>(y),
                       static_cast<const T*>(up), static_cast<T*>(dst), rows, cols);
  else
    hipLaunchKernelGGL((softmax_grad_rows_kernel<T, 1>), grid, dim3(256), 0, s, static_cast<const T*>(y),
                       static_cast<const T*>(up), static_cast<T*>(dst), rows, cols);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T>
static int argmax_typed(const void* a, void* dst, int64_t outer, int64_t reduce, int64_t inner, hipStream_t s) {
  if (inner == 1)
    hipLaunchKernelGGL((argmax_last_kernel<T>), dim3(static_cast<unsigned>(ceil_div(outer, 4))), dim3(256), 0, s,
                       static_cast<const T*>(a), static_cast<T*>(dst), outer, reduce);
  else
    hipLaunchKernelGGL((argmax_mid_kernel<T>), dim3(static_cast<unsigned>(ceil_div(outer * inner, 256))), dim3(256), 0, s,
                       static_cast<const T*>(a), static_cast<T*>(dst), outer, reduce, inner);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

static int check_rows(const char* who, int64_t rows, int64_t cols, int dtype) {
  if (!is_float_dtype(dtype)) return fail(MG_ERR_INVALID, "%s: unsupported dtype %s", who, dtype_name(dtype));
  if (rows < 0 || cols < 0) return fail(MG_ERR_INVALID, "%s: negative shape", who);
  if (rows > int64_t{4} * 0x7fffffff) return fail(MG_ERR_UNSUPPORTED, "%s: too many rows", who);
  return MG_OK;
}

}  // namespace mg

extern "C" {

int mg_softmax(const void* x, void* y, int64_t rows, int64_t cols, int dtype, mg_stream stream) {
  MG_TRY(mg::check_rows("softmax", rows, cols, dtype));
  if (rows == 0 || cols == 0) return MG_OK;
  if (!x || !y) return mg::fail(MG_ERR_INVALID, "softmax: null pointer argument");
  hipStream_t s = mg::to_stream(stream);
  switch (dtype) {
    case MG_F32: return mg::softmax_typed<float>(x, y, rows, cols, s);
    case MG_F16: return mg::softmax_typed<mg::f16_t>(x, y, rows, cols, s);
    default: return mg::softmax_typed<mg::bf16_t>(x, y, rows, cols, s);
  }
}

int mg_softmax_strided(const void* x, void* y, int rank, const int64_t* shape, const int64_t* strides, int dtype,
                       mg_stream stream) {
  if (rank < 1 || rank > mg::kMaxRank)
    return mg::fail(MG_ERR_INVALID, "softmax_strided: rank %d outside 1..%d", rank, mg::kMaxRank);
  if (!shape || !strides) return mg::fail(MG_ERR_INVALID, "softmax_strided: null shape or strides");
  int64_t rows = 1;
  mg::StridedView v;
  v.rank = rank - 1;
  for (int d = 0; d < rank; ++d) {
    if (shape[d] < 0 || strides[d] < 0)
      return mg::fail(MG_ERR_INVALID, "softmax_strided: negative extent or stride at dim %d", d);
    if (d + 1 < rank) {
      rows *= shape[d];
      v.shape[d] = shape[d];
      v.stride[d] = strides[d];
    }
  }
  const int64_t cols = shape[rank - 1], xs = strides[rank - 1];
  MG_TRY(mg::check_rows("softmax_strided", rows, cols, dtype));
  if (rows == 0 || cols == 0) return MG_OK;
  if (!x || !y) return mg::fail(MG_ERR_INVALID, "softmax_strided: null pointer argument");
  // Rows that run across memory lines (a transposed view) of a large tensor: copy the view
  // row-major first (mg_contiguous moves transposes through LDS tiles) and take the flat kernel.
  if (xs > 1 && cols >= 32 && rows * cols >= (int64_t{1} << 16)) {
    bool has_unit = false;
    for (int d = 0; d + 1 < rank; ++d) has_unit = has_unit || (strides[d] == 1 && shape[d] >= 32);
    if (has_unit) {
      mg::Scratch copy;
      MG_TRY(copy.take(rows * cols * static_cast<int64_t>(mg::dtype_size(dtype))));
      MG_TRY(mg_contiguous(x, copy.as<char>(), rank, shape, strides, dtype, stream));
      return mg_softmax(copy.as<char>(), y, rows, cols, dtype, stream);
    }
  }
  // 16-byte loads where a row is contiguous and every row starts on a 16-byte boundary
  bool wide = xs == 1 && mg::aligned16(x) && mg::aligned16(y);
  for (int d = 0; d + 1 < rank && wide; ++d) wide = shape[d] == 1 || strides[d] * mg::dtype_size(dtype) % 16 == 0;
  hipStream_t s = mg::to_stream(stream);
  switch (dtype) {
    case MG_F32: return mg::softmax_view_typed<float>(x, y, v, xs, rows, cols, wide, s);
    case MG_F16: return mg::softmax_view_typed<mg::f16_t>(x, y, v, xs, rows, cols, wide, s);
    default: return mg::softmax_view_typed<mg::bf16_t>(x, y, v, xs, rows, cols, wide, s);
  }
}

int mg_softmax_grad(const void* y, const void* upstream, void* dst, int64_t rows, int64_t cols, int dtype,
                    mg_stream stream) {
  MG_TRY(mg::check_rows("softmax_grad", rows, cols, dtype));
  if (rows == 0 || cols == 0) return MG_OK;
  if (!y || !upstream || !dst) return mg::fail(MG_ERR_INVALID, "softmax_grad: null pointer argument");
  hipStream_t s = mg::to_stream(stream);
  switch (dtype) {
    case MG_F32: return mg::softmax_grad_typed<float>(y, upstream, dst, rows, cols, s);
    case MG_F16: return mg::softmax_grad_typed<mg::f16_t>(y, upstream, dst, rows, cols, s);
    default: return mg::softmax_grad_typed<mg::bf16_t>(y, upstream, dst, rows, cols, s);
  }
}

int mg_argmax_axis(const void* a, void* dst, int64_t outer, int64_t reduce, int64_t inner, int dtype, mg_stream stream) {
  if (!mg::is_float_dtype(dtype)) return mg::fail(MG_ERR_INVALID, "argmax: unsupported dtype %s", mg::dtype_name(dtype));
  if (outer < 0 || reduce < 0 || inner < 0) return mg::fail(MG_ERR_INVALID, "argmax: negative shape");
  if (outer == 0 || inner == 0) return MG_OK;
  if (!dst || (reduce > 0 && !a)) return mg::fail(MG_ERR_INVALID, "argmax: null pointer argument");
  hipStream_t s = mg::to_stream(stream);
  switch (dtype) {
    case MG_F32: return mg::argmax_typed<float>(a, dst, outer, reduce, inner, s);
    case MG_F16: return mg::argmax_typed<mg::f16_t>(a, dst, outer, reduce, inner, s);
    default: return mg::argmax_typed<mg::bf16_t>(a, dst, outer, reduce, inner, s);
  }
}

}  // extern "C"
