// Elementwise maps of the training step around the backward kernels: residual and gradient
// adds, relu, dtype casts, and the copy that makes a strided view contiguous, plus the same
// maps over strided (transposed, sliced, broadcast) views.  All are HBM-bound streaming kernels
// with 16-byte accesses where the views allow them.
#include "mg_device.h"
#include "mg_internal.h"

namespace mg {

template <typename T>
__global__ __launch_bounds__(256) void add_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ dst,
                                                  int64_t n) {
  constexpr int VEC = WideVec<T>::value;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * VEC;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * VEC; i < n; i += stride) {
    if (i + VEC <= n) {
      float x[VEC], y[VEC];
      VecIO<T, VEC>::load(a + i, x);
      VecIO<T, VEC>::load(b + i, y);
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[e] += y[e];
      VecIO<T, VEC>::store_stream(dst + i, x);
    } else {
      for (int64_t j = i; j < n; ++j) dst[j] = from_float<T>(to_float(a[j]) + to_float(b[j]));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void relu_kernel(const T* __restrict__ a, T* __restrict__ dst, int64_t n) {
  constexpr int VEC = WideVec<T>::value;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * VEC;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * VEC; i < n; i += stride) {
    if (i + VEC <= n) {
      float x[VEC];
      VecIO<T, VEC>::load(a + i, x);
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[e] = x[e] > 0.f ? x[e] : 0.f;
      VecIO<T, VEC>::store_stream(dst + i, x);
    } else {
      for (int64_t j = i; j < n; ++j) dst[j] = to_float(a[j]) > 0.f ? a[j] : from_float<T>(0.f);
    }
  }
}

// Eight elements per thread: two 16-byte accesses on the fp32 side, one on the 16-bit side.
template <typename S, typename D>
__global__ __launch_bounds__(256) void cast_kernel(const S* __restrict__ a, D* __restrict__ dst, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256 * 8;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 8; i < n; i += stride) {
    if (i + 8 <= n) {
      float v[8];
      if constexpr (sizeof(S) == 4) {
        float lo[4], hi[4];
        VecIO<S, 4>::load(a + i, lo);
        VecIO<S, 4>::load(a + i + 4, hi);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = lo[e];
          v[4 + e] = hi[e];
        }
      } else {
        VecIO<S, 8>::load(a + i, v);
      }
      if constexpr (sizeof(D) == 4) {
        const float lo[4] = {v[0], v[1], v[2], v[3]};
        const float hi[4] = {v[4], v[5], v[6], v[7]};
        VecIO<D, 4>::store(dst + i, lo);
        VecIO<D, 4>::store(dst + i + 4, hi);
      } else {
        VecIO<D, 8>::store(dst + i, v);
      }
    } else {
      for (int64_t j = i; j < n; ++j) dst[j] = from_float<D>(to_float(a[j]));
    }
  }
}

// dst[flat] = src[offset(flat)] over chunks of sizeof(V) bytes.  The view's shape and
// strides are in chunk units; flat runs over the row-major order of the shape.  Index is
// uint32_t when every extent and offset fits, else int64_t.
struct CopyView {
  int rank;
  int64_t shape[kMaxRank];
  int64_t stride[kMaxRank];
};

template <typename V, typename Index>
__global__ __launch_bounds__(256) void contiguous_kernel(const V* __restrict__ src, V* __restrict__ dst, CopyView v,
                                                         int64_t n) {
  const int64_t step = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t flat = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; flat < n; flat += step) {
    Index rem = static_cast<Index>(flat);
    Index off = 0;
    for (int d = v.rank - 1; d > 0; --d) {
      const Index extent = static_cast<Index>(v.shape[d]);
      const Index q = rem / extent;
      off += (rem - q * extent) * static_cast<Index>(v.stride[d]);
      rem = q;
    }
    off += rem * static_cast<Index>(v.stride[0]);
    dst[flat] = src[off];
  }
}

// ---- the same maps over strided views -----------------------------------------------------
// dst (row-major) = op(a[view a], b[view b]): both operands are views of dst's shape with their
// own element strides (0 along a broadcast axis).  A thread takes VEC consecutive elements of
// the innermost axis; an operand whose innermost stride is 1 is read with 16-byte loads, one
// whose innermost stride is 0 is read once and repeated; VEC = 1 serves every other view
// element by element.  `shape` holds the innermost extent in units of VEC, `sa`/`sb` the
// innermost strides times VEC.
enum MapOp { kMapAdd = 0, kMapRelu = 1, kMapReluGrad = 2, kMapCast = 3 };

struct MapView {
  int rank;
  int64_t shape[kMaxRank];
  int64_t sa[kMaxRank];
  int64_t sb[kMaxRank];
};

// Elements per thread of the wide form: one 16-byte access on each side, two on the fp32 side
// of a cast to or from 16 bits.
template <typename S, typename D>
struct MapWide {
  static constexpr int value = sizeof(S) == 4 && sizeof(D) == 4 ? 4 : 8;
};

template <typename T, int VEC>
__device__ __forceinline__ void map_load(const T* __restrict__ p, bool unit, float (&v)[VEC]) {
  if constexpr (VEC == 1) {
    v[0] = to_float(*p);
  } else if (unit) {
    if constexpr (sizeof(T) == 4 && VEC == 8) {
      float lo[4], hi[4];
      VecIO<T, 4>::load(p, lo);
      VecIO<T, 4>::load(p + 4, hi);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] = lo[e];
        v[4 + e] = hi[e];
      }
    } else {
      VecIO<T, VEC>::load(p, v);
    }
  } else {
    const float x = to_float(*p);
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = x;
  }
}

template <typename T, int VEC>
__device__ __forceinline__ void map_store(T* __restrict__ p, const float (&v)[VEC]) {
  if constexpr (VEC == 1) {
    *p = from_float<T>(v[0]);
  } else if constexpr (sizeof(T) == 4 && VEC == 8) {
    const float lo[4] = {v[0], v[1], v[2], v[3]};
    const float hi[4] = {v[4], v[5], v[6], v[7]};
    VecIO<T, 4>::store(p, lo);
    VecIO<T, 4>::store(p + 4, hi);
  } else {
    VecIO<T, VEC>::store(p, v);
  }
}

template <typename S, typename D, int OP, int VEC, typename Index>
__global__ __launch_bounds__(256) void map_strided_kernel(const S* __restrict__ a, const S* __restrict__ b,
                                                          D* __restrict__ dst, MapView v, int64_t n, bool a_unit,
                                                          bool b_unit) {
  constexpr bool kBinary = OP == kMapAdd || OP == kMapReluGrad;
  const int64_t step = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t flat = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; flat < n; flat += step) {
    Index rem = static_cast<Index>(flat);
    Index off_a = 0, off_b = 0;
    for (int d = v.rank - 1; d > 0; --d) {
      const Index extent = static_cast<Index>(v.shape[d]);
      const Index q = rem / extent;
      const Index idx = rem - q * extent;
      off_a += idx * static_cast<Index>(v.sa[d]);
      if constexpr (kBinary) off_b += idx * static_cast<Index>(v.sb[d]);
      rem = q;
    }
    off_a += rem * static_cast<Index>(v.sa[0]);
    if constexpr (kBinary) off_b += rem * static_cast<Index>(v.sb[0]);
    float x[VEC], y[VEC];
    map_load<S, VEC>(a + off_a, a_unit, x);
    if constexpr (kBinary) map_load<S, VEC>(b + off_b, b_unit, y);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      if constexpr (OP == kMapAdd) x[e] += y[e];
      else if constexpr (OP == kMapRelu) x[e] = x[e] > 0.f ? x[e] : 0.f;
      else if constexpr (OP == kMapReluGrad) x[e] = x[e] > 0.f ? y[e] : 0.f;
    }
    map_store<D, VEC>(dst + flat * VEC, x);
  }
}

// The same copy for a view whose innermost dim is strided while another dim is contiguous in the
// source (a transpose, possibly with outer dims around and between): TILE x TILE elements go
// through LDS, read along the source's contiguous dim and written along the result's, so both
// sides move whole cache lines where the element-wise kernel reads one element per line.
// `col` is the source-contiguous dim (stride 1), `row` the innermost dim of the result; the
// other dims are batch dims, decomposed per workgroup.
struct TransposeView {
  int nbatch;                  // batch dims
  int64_t bshape[kMaxRank];    // their extents, outermost first
  int64_t bsrc[kMaxRank];      // their source strides (elements)
  int64_t bdst[kMaxRank];      // their strides in the result
  int64_t rows, cols;          // extents of the two transposed dims
  int64_t row_src_stride;      // source stride of the row dim
  int64_t col_dst_stride;      // stride of the col dim in the result
};

template <typename V, int TILE>
__global__ __launch_bounds__(256) void contiguous_transpose_kernel(const V* __restrict__ src, V* __restrict__ dst,
                                                                   TransposeView v, int64_t col_tiles,
                                                                   int64_t row_tiles) {
  constexpr int TY = 256 / TILE;
  __shared__ V tile[TILE][TILE + 1];
  int64_t w = blockIdx.x;
  const int64_t ct = w % col_tiles;
  w /= col_tiles;
  const int64_t rt = w % row_tiles;
  w /= row_tiles;
  int64_t src_at = 0, dst_at = 0;
  for (int d = v.nbatch - 1; d >= 0; --d) {
    const int64_t q = w / v.bshape[d], i = w - q * v.bshape[d];
    src_at += i * v.bsrc[d];
    dst_at += i * v.bdst[d];
    w = q;
  }
  const int tx = threadIdx.x % TILE, ty = threadIdx.x / TILE;
  const int64_t c0 = ct * TILE, r0 = rt * TILE;
#pragma unroll
  for (int k = 0; k < TILE; k += TY) {
    const int64_t r = r0 + ty + k, c = c0 + tx;
    if (r < v.rows && c < v.cols) tile[ty + k][tx] = src[src_at + r * v.row_src_stride + c];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < TILE; k += TY) {
    const int64_t c = c0 + ty + k, r = r0 + tx;
    if (r < v.rows && c < v.cols) dst[dst_at + c * v.col_dst_stride + r] = tile[tx][ty + k];
  }
}

static unsigned stream_blocks(int64_t n, int per_thread) {
  int64_t blocks = ceil_div(n, static_cast<int64_t>(256) * per_thread);
  const int64_t cap = static_cast<int64_t>(device_info().cu_count) * 16;
  if (blocks > cap) blocks = cap;
  return static_cast<unsigned>(blocks < 1 ? 1 : blocks);
}

template <typename T>
static int add_typed(const void* a, const void* b, void* dst, int64_t n, hipStream_t s) {
  hipLaunchKernelGGL((add_kernel<T>), dim3(stream_blocks(n, WideVec<T>::value)), dim3(256), 0, s,
                     static_cast<const T*>(a), static_cast<const T*>(b), static_cast<T*>(dst), n);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T>
static int relu_typed(const void* a, void* dst, int64_t n, hipStream_t s) {
  hipLaunchKernelGGL((relu_kernel<T>), dim3(stream_blocks(n, WideVec<T>::value)), dim3(256), 0, s,
                     static_cast<const T*>(a), static_cast<T*>(dst), n);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename S, typename D>
static int cast_typed(const void* a, void* dst, int64_t n, hipStream_t s) {
  hipLaunchKernelGGL((cast_kernel<S, D>), dim3(stream_blocks(n, 8)), dim3(256), 0, s, static_cast<const S*>(a),
                     static_cast<D*>(dst), n);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename S>
static int cast_from(const void* a, void* dst, int64_t n, int out_dtype, hipStream_t s) {
  switch (out_dtype) {
    case MG_F32: return cast_typed<S, float>(a, dst, n, s);
    case MG_F16: return cast_typed<S, f16_t>(a, dst, n, s);
    default: return cast_typed<S, bf16_t>(a, dst, n, s);
  }
}

template <typename V>
static int contiguous_launch(const void* src, void* dst, const CopyView& v, int64_t n, bool narrow, hipStream_t s) {
  const dim3 grid(stream_blocks(n, 1));
  if (narrow)
    hipLaunchKernelGGL((contiguous_kernel<V, uint32_t>), grid, dim3(256), 0, s, static_cast<const V*>(src),
                       static_cast<V*>(dst), v, n);
  else
    hipLaunchKernelGGL((contiguous_kernel<V, int64_t>), grid, dim3(256), 0, s, static_cast<const V*>(src),
                       static_cast<V*>(dst), v, n);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

// The tiled transpose for normalised dims (sh, st): taken when the innermost dim is strided, one
// other dim has stride 1, and both are long enough to fill tiles.  Returns false when the view is
// not of that kind (kNotTransposed), else the launch's status.
constexpr int kNotTransposed = -1;
template <typename V, int TILE>
static int contiguous_transpose_try(const void* src, void* dst, int r, const int64_t* sh, const int64_t* st,
                                    hipStream_t s) {
  if (r < 2 || st[r - 1] == 1 || st[r - 1] == 0) return kNotTransposed;
  int p = -1;
  for (int d = 0; d + 1 < r; ++d)
    if (st[d] == 1) p = d;
  if (p < 0 || sh[p] < TILE / 2 || sh[r - 1] < TILE / 2) return kNotTransposed;
  int64_t dstride[kMaxRank];
  dstride[r - 1] = 1;
  for (int d = r - 2; d >= 0; --d) dstride[d] = dstride[d + 1] * sh[d + 1];
  TransposeView v;
  v.nbatch = 0;
  int64_t batch = 1;
  for (int d = 0; d + 1 < r; ++d) {
    if (d == p) continue;
    v.bshape[v.nbatch] = sh[d];
    v.bsrc[v.nbatch] = st[d];
    v.bdst[v.nbatch] = dstride[d];
    ++v.nbatch;
    batch *= sh[d];
  }
  v.rows = sh[r - 1];
  v.cols = sh[p];
  v.row_src_stride = st[r - 1];
  v.col_dst_stride = dstride[p];
  const int64_t col_tiles = ceil_div(v.cols, TILE), row_tiles = ceil_div(v.rows, TILE);
  const int64_t blocks = col_tiles * row_tiles * batch;
  if (blocks > 0x7fffffffLL) return kNotTransposed;
  hipLaunchKernelGGL((contiguous_transpose_kernel<V, TILE>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s,
                     static_cast<const V*>(src), static_cast<V*>(dst), v, col_tiles, row_tiles);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

static int contiguous_dispatch(const void* src, void* dst, int rank, const int64_t* shape, const int64_t* strides,
                               int dtype, hipStream_t s) {
  const int esz = dtype_size(dtype);
  if (esz == 0) return fail(MG_ERR_INVALID, "contiguous: unsupported dtype %d", dtype);
  if (rank < 0 || rank > kMaxRank) return fail(MG_ERR_INVALID, "contiguous: rank %d outside 0..%d", rank, kMaxRank);
  if (rank > 0 && (!shape || !strides)) return fail(MG_ERR_INVALID, "contiguous: null shape or strides");
  int64_t n = 1;
  for (int d = 0; d < rank; ++d) {
    if (shape[d] < 0 || strides[d] < 0)
      return fail(MG_ERR_INVALID, "contiguous: negative extent or stride at dim %d", d);
    n *= shape[d];
  }
  if (n == 0) return MG_OK;
  if (!src || !dst) return fail(MG_ERR_INVALID, "contiguous: null pointer argument");
  // Drop unit dims and merge neighbours that are contiguous with each other.
  int64_t sh[kMaxRank], st[kMaxRank];
  int r = 0;
  for (int d = 0; d < rank; ++d) {
    if (shape[d] == 1) continue;
    if (r > 0 && st[r - 1] == shape[d] * strides[d]) {
      sh[r - 1] *= shape[d];
      st[r - 1] = strides[d];
    } else {
      sh[r] = shape[d];
      st[r] = strides[d];
      ++r;
    }
  }
  if (r == 0) {
    sh[0] = 1;
    st[0] = 1;
    r = 1;
  }
  if (env_int("MOGRAD_HIP_CONTIGUOUS_TRANSPOSE", 1) != 0) {  // transposes go through LDS tiles
    int status = kNotTransposed;
    switch (esz) {
      case 8: status = contiguous_transpose_try<uint2, 32>(src, dst, r, sh, st, s); break;
      case 4: status = contiguous_transpose_try<uint32_t, 32>(src, dst, r, sh, st, s); break;
      case 2: status = contiguous_transpose_try<uint16_t, 64>(src, dst, r, sh, st, s); break;
      default: break;
    }
    if (status != kNotTransposed) return status;
  }
  // Widest chunk (bytes) that divides the innermost run and every outer stride.
  int chunk = esz;
  if (st[r - 1] == 1) {
    for (int c = 16; c > esz; c /= 2) {
      const int64_t elems = c / esz;
      bool ok = sh[r - 1] % elems == 0 && reinterpret_cast<uintptr_t>(src) % c == 0 &&
                reinterpret_cast<uintptr_t>(dst) % c == 0;
      for (int d = 0; d + 1 < r && ok; ++d) ok = st[d] % elems == 0;
      if (ok) {
        chunk = c;
        break;
      }
    }
  }
  const int64_t elems = chunk / esz;
  CopyView v;
  v.rank = r;
  int64_t max_off = 0;
  for (int d = 0; d < r; ++d) {
    v.shape[d] = d == r - 1 ? sh[d] / elems : sh[d];
    v.stride[d] = d == r - 1 ? st[d] : st[d] / elems;  // innermost stride is 1 chunk when elems > 1
    max_off += (v.shape[d] - 1) * v.stride[d];
  }
  const int64_t chunks = n / elems;
  const bool narrow = chunks < (int64_t{1} << 31) && max_off < (int64_t{1} << 31);
  switch (chunk) {
    case 16: return contiguous_launch<uint4>(src, dst, v, chunks, narrow, s);
    case 8: return contiguous_launch<uint2>(src, dst, v, chunks, narrow, s);
    case 4: return contiguous_launch<uint32_t>(src, dst, v, chunks, narrow, s);
    default: return contiguous_launch<uint16_t>(src, dst, v, chunks, narrow, s);
  }
}

template <typename S, typename D, int OP>
static int map_strided_typed(const void* a, const void* b, void* dst, const MapView& v, int64_t n, int vec, bool narrow,
                             bool a_unit, bool b_unit, hipStream_t s) {
  const dim3 grid(stream_blocks(n, 1));
  const S* pa = static_cast<const S*>(a);
  const S* pb = static_cast<const S*>(b);
  D* pd = static_cast<D*>(dst);
#define MG_MAP_LAUNCH(VEC_, INDEX_) \
  hipLaunchKernelGGL((map_strided_kernel<S, D, OP, VEC_, INDEX_>), grid, dim3(256), 0, s, pa, pb, pd, v, n, a_unit, b_unit)
  if (vec > 1) {
    constexpr int kWide = MapWide<S, D>::value;
    if (narrow) MG_MAP_LAUNCH(kWide, uint32_t);
    else MG_MAP_LAUNCH(kWide, int64_t);
  } else {
    if (narrow) MG_MAP_LAUNCH(1, uint32_t);
    else MG_MAP_LAUNCH(1, int64_t);
  }
#undef MG_MAP_LAUNCH
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <int OP>
static int map_strided_dtypes(const void* a, const void* b, void* dst, const MapView& v, int64_t n, int vec, bool narrow,
                              bool a_unit, bool b_unit, int in_dtype, int out_dtype, hipStream_t s) {
#define MG_MAP_TYPED(S_, D_) return map_strided_typed<S_, D_, OP>(a, b, dst, v, n, vec, narrow, a_unit, b_unit, s)
  if constexpr (OP == kMapCast) {
    if (in_dtype == MG_F32) {
      if (out_dtype == MG_F32) MG_MAP_TYPED(float, float);
      if (out_dtype == MG_F16) MG_MAP_TYPED(float, f16_t);
      MG_MAP_TYPED(float, bf16_t);
    }
    if (in_dtype == MG_F16) {
      if (out_dtype == MG_F32) MG_MAP_TYPED(f16_t, float);
      if (out_dtype == MG_F16) MG_MAP_TYPED(f16_t, f16_t);
      MG_MAP_TYPED(f16_t, bf16_t);
    }
    if (out_dtype == MG_F32) MG_MAP_TYPED(bf16_t, float);
    if (out_dtype == MG_F16) MG_MAP_TYPED(bf16_t, f16_t);
    MG_MAP_TYPED(bf16_t, bf16_t);
  } else {
    if (in_dtype == MG_F32) MG_MAP_TYPED(float, float);
    if (in_dtype == MG_F16) MG_MAP_TYPED(f16_t, f16_t);
    MG_MAP_TYPED(bf16_t, bf16_t);
  }
#undef MG_MAP_TYPED
}

// Checks the views, drops unit dims, merges neighbours that are contiguous with each other in
// both operands, picks 4 or 8 elements per thread where every operand allows it, and launches.
template <int OP>
static int map_strided_dispatch(const char* who, const void* a, const void* b, void* dst, int rank, const int64_t* shape,
                                const int64_t* strides_a, const int64_t* strides_b, int in_dtype, int out_dtype,
                                hipStream_t s) {
  constexpr bool kBinary = OP == kMapAdd || OP == kMapReluGrad;
  if (!is_float_dtype(in_dtype) || !is_float_dtype(out_dtype))
    return fail(MG_ERR_INVALID, "%s: unsupported dtype %s", who,
                dtype_name(is_float_dtype(in_dtype) ? out_dtype : in_dtype));
  if (rank < 0 || rank > kMaxRank) return fail(MG_ERR_INVALID, "%s: rank %d outside 0..%d", who, rank, kMaxRank);
  if (rank > 0 && (!shape || !strides_a || (kBinary && !strides_b)))
    return fail(MG_ERR_INVALID, "%s: null shape or strides", who);
  int64_t n = 1;
  for (int d = 0; d < rank; ++d) {
    if (shape[d] < 0 || strides_a[d] < 0 || (kBinary && strides_b[d] < 0))
      return fail(MG_ERR_INVALID, "%s: negative extent or stride at dim %d", who, d);
    n *= shape[d];
  }
  if (n == 0) return MG_OK;
  if (!a || (kBinary && !b) || !dst) return fail(MG_ERR_INVALID, "%s: null pointer argument", who);
  // A large operand that is a transpose (innermost dim strided, another dim contiguous in memory)
  // would be read one element per cache line: it is first copied row-major through the tiled
  // transpose (3-5 x the rate of the element-wise read) and the map then runs on the copy.
  Scratch copy_a, copy_b;
  int64_t row_major[kMaxRank];
  {
    int64_t run = 1;
    for (int d = rank - 1; d >= 0; --d) {
      row_major[d] = run;
      run *= shape[d];
    }
  }
  auto transposed = [&](const int64_t* st) {
    if (n < (int64_t{1} << 16) || env_int("MOGRAD_HIP_CONTIGUOUS_TRANSPOSE", 1) == 0) return false;
    int inner = rank - 1;
    while (inner >= 0 && shape[inner] == 1) --inner;
    if (inner < 0 || st[inner] <= 1 || shape[inner] < 32) return false;
    for (int d = 0; d < inner; ++d)
      if (st[d] == 1 && shape[d] >= 32) return true;
    return false;
  };
  if (transposed(strides_a)) {
    MG_TRY(copy_a.take(n * static_cast<int64_t>(dtype_size(in_dtype))));
    MG_TRY(contiguous_dispatch(a, copy_a.as<char>(), rank, shape, strides_a, in_dtype, s));
    a = copy_a.as<char>();
    strides_a = row_major;
  }
  if (kBinary && transposed(strides_b)) {
    MG_TRY(copy_b.take(n * static_cast<int64_t>(dtype_size(in_dtype))));
    MG_TRY(contiguous_dispatch(b, copy_b.as<char>(), rank, shape, strides_b, in_dtype, s));
    b = copy_b.as<char>();
    strides_b = row_major;
  }
  int64_t sh[kMaxRank], sa[kMaxRank], sb[kMaxRank];
  int r = 0;
  for (int d = 0; d < rank; ++d) {
    if (shape[d] == 1) continue;
    const int64_t tb = kBinary ? strides_b[d] : 0;
    if (r > 0 && sa[r - 1] == shape[d] * strides_a[d] && sb[r - 1] == shape[d] * tb) {
      sh[r - 1] *= shape[d];
      sa[r - 1] = strides_a[d];
      sb[r - 1] = tb;
    } else {
      sh[r] = shape[d];
      sa[r] = strides_a[d];
      sb[r] = tb;
      ++r;
    }
  }
  if (r == 0) {
    sh[0] = 1;
    sa[0] = sb[0] = 1;
    r = 1;
  }
  // A group per thread: the innermost extent in whole groups, dst and every unit-stride operand
  // on 16-byte boundaries at every group (base pointer and outer strides), any other operand
  // constant along the innermost axis.
  const int in_size = dtype_size(in_dtype);
  auto wide_operand = [&](const void* p, const int64_t* st) {
    if (st[r - 1] == 0) return true;
    if (st[r - 1] != 1 || !aligned16(p)) return false;
    for (int d = 0; d + 1 < r; ++d)
      if (st[d] * in_size % 16 != 0) return false;
    return true;
  };
  const int group = dtype_size(in_dtype) == 4 && dtype_size(out_dtype) == 4 ? 4 : 8;  // MapWide
  const bool wide = sh[r - 1] % group == 0 && aligned16(dst) && wide_operand(a, sa) && (!kBinary || wide_operand(b, sb));
  const int vec = wide ? group : 1;
  MapView v;
  v.rank = r;
  int64_t max_a = 0, max_b = 0;
  for (int d = 0; d < r; ++d) {
    const bool inner = d == r - 1;
    v.shape[d] = inner ? sh[d] / vec : sh[d];
    v.sa[d] = inner ? sa[d] * vec : sa[d];
    v.sb[d] = inner ? sb[d] * vec : sb[d];
    max_a += (v.shape[d] - 1) * v.sa[d];
    max_b += (v.shape[d] - 1) * v.sb[d];
  }
  const int64_t chunks = n / vec;
  const bool narrow = n < (int64_t{1} << 31) && max_a < (int64_t{1} << 31) && max_b < (int64_t{1} << 31);
  return map_strided_dtypes<OP>(a, b, dst, v, chunks, vec, narrow, sa[r - 1] == 1, sb[r - 1] == 1, in_dtype, out_dtype, s);
}

}  // namespace mg

extern "C" {

int mg_add(const void* a, const void* b, void* dst, int64_t n, int dtype, mg_stream stream) {
  if (!mg::is_float_dtype(dtype)) return mg::fail(MG_ERR_INVALID, "add: unsupported dtype %s", mg::dtype_name(dtype));
  if (n < 0) return mg::fail(MG_ERR_INVALID, "add: negative size");
  if (n == 0) return MG_OK;
  if (!a || !b || !dst) return mg::fail(MG_ERR_INVALID, "add: null pointer argument");
  if (!mg::aligned16(a) || !mg::aligned16(b) || !mg::aligned16(dst))
    return mg::fail(MG_ERR_INVALID, "add: pointers must be 16-byte aligned");
  hipStream_t s = mg::to_stream(stream);
  switch (dtype) {
    case MG_F32: return mg::add_typed<float>(a, b, dst, n, s);
    case MG_F16: return mg::add_typed<mg::f16_t>(a, b, dst, n, s);
    default: return mg::add_typed<mg::bf16_t>(a, b, dst, n, s);
  }
}

int mg_relu(const void* a, void* dst, int64_t n, int dtype, mg_stream stream) {
  if (!mg::is_float_dtype(dtype)) return mg::fail(MG_ERR_INVALID, "relu: unsupported dtype %s", mg::dtype_name(dtype));
  if (n < 0) return mg::fail(MG_ERR_INVALID, "relu: negative size");
  if (n == 0) return MG_OK;
  if (!a || !dst) return mg::fail(MG_ERR_INVALID, "relu: null pointer argument");
  if (!mg::aligned16(a) || !mg::aligned16(dst)) return mg::fail(MG_ERR_INVALID, "relu: pointers must be 16-byte aligned");
  hipStream_t s = mg::to_stream(stream);
  switch (dtype) {
    case MG_F32: return mg::relu_typed<float>(a, dst, n, s);
    case MG_F16: return mg::relu_typed<mg::f16_t>(a, dst, n, s);
    default: return mg::relu_typed<mg::bf16_t>(a, dst, n, s);
  }
}

int mg_cast(const void* a, void* dst, int64_t n, int in_dtype, int out_dtype, mg_stream stream) {
  if (!mg::is_float_dtype(in_dtype) || !mg::is_float_dtype(out_dtype))
    return mg::fail(MG_ERR_INVALID, "cast: unsupported dtype combination %s -> %s", mg::dtype_name(in_dtype),
                    mg::dtype_name(out_dtype));
  if (n < 0) return mg::fail(MG_ERR_INVALID, "cast: negative size");
  if (n == 0) return MG_OK;
  if (!a || !dst) return mg::fail(MG_ERR_INVALID, "cast: null pointer argument");
  if (!mg::aligned16(a) || !mg::aligned16(dst)) return mg::fail(MG_ERR_INVALID, "cast: pointers must be 16-byte aligned");
  hipStream_t s = mg::to_stream(stream);
  if (in_dtype == out_dtype) {
    MG_HIP(hipMemcpyAsync(dst, a, static_cast<size_t>(n) * mg::dtype_size(in_dtype), hipMemcpyDeviceToDevice, s));
    return MG_OK;
  }
  switch (in_dtype) {
    case MG_F32: return mg::cast_from<float>(a, dst, n, out_dtype, s);
    case MG_F16: return mg::cast_from<mg::f16_t>(a, dst, n, out_dtype, s);
    default: return mg::cast_from<mg::bf16_t>(a, dst, n, out_dtype, s);
  }
}

int mg_contiguous(const void* a, void* dst, int rank, const int64_t* shape, const int64_t* strides, int dtype,
                  mg_stream stream) {
  return mg::contiguous_dispatch(a, dst, rank, shape, strides, dtype, mg::to_stream(stream));
}

int mg_add_strided(const void* a, const void* b, void* dst, int rank, const int64_t* shape, const int64_t* strides_a,
                   const int64_t* strides_b, int dtype, mg_stream stream) {
  return mg::map_strided_dispatch<mg::kMapAdd>("add_strided", a, b, dst, rank, shape, strides_a, strides_b, dtype, dtype,
                                               mg::to_stream(stream));
}

int mg_relu_strided(const void* a, void* dst, int rank, const int64_t* shape, const int64_t* strides, int dtype,
                    mg_stream stream) {
  return mg::map_strided_dispatch<mg::kMapRelu>("relu_strided", a, nullptr, dst, rank, shape, strides, nullptr, dtype, dtype,
                                                mg::to_stream(stream));
}

int mg_relu_grad_strided(const void* out, const void* upstream, void* dst, int rank, const int64_t* shape,
                         const int64_t* strides_out, const int64_t* strides_upstream, int dtype, mg_stream stream) {
  return mg::map_strided_dispatch<mg::kMapReluGrad>("relu_grad_strided", out, upstream, dst, rank, shape, strides_out,
                                                    strides_upstream, dtype, dtype, mg::to_stream(stream));
}

int mg_cast_strided(const void* a, void* dst, int rank, const int64_t* shape, const int64_t* strides, int in_dtype,
                    int out_dtype, mg_stream stream) {
  return mg::map_strided_dispatch<mg::kMapCast>("cast_strided", a, nullptr, dst, rank, shape, strides, nullptr, in_dtype,
                                                out_dtype, mg::to_stream(stream));
}

}  // extern "C"
