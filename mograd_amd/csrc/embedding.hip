// Row gather (embedding lookup) and its gradient, the row scatter-add.
//
// The scatter-add uses no atomics: each wave owns one destination row (and one slab of
// the index list), scans the indices 64 at a time, and adds the matching value rows in
// index order with fp32 accumulation, so the result does not depend on scheduling.
// That costs rows x indices comparisons, fine for a 65-row table and hopeless for a 50304-row
// one; large tables first sort (row, position) pairs by row (a stable radix sort, so
// positions stay ascending inside a row), and a wave then adds only its own row's run.
#include <algorithm>
#include <cstring>
#include <utility>

#include "mg_device.h"
#include "mg_internal.h"
#include "mg_rows.h"

namespace mg {

// dst(i, :) = src(indices[i], :) over chunks of VEC elements; rows whose index is outside
// [0, num_rows) are filled with zeros.
template <typename T, typename I, int VEC>
__global__ __launch_bounds__(256) void gather_rows_kernel(const T* __restrict__ src, const I* __restrict__ indices,
                                                          T* __restrict__ dst, int64_t n_idx, int64_t num_rows,
                                                          int64_t row_size, int64_t row_stride, int64_t col_stride) {
  const int64_t chunks_per_row = row_size / VEC;
  const int64_t total = n_idx * chunks_per_row;
  const int64_t step = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t flat = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; flat < total; flat += step) {
    const int64_t i = flat / chunks_per_row;
    const int64_t c = (flat - i * chunks_per_row) * VEC;
    const int64_t r = static_cast<int64_t>(indices[i]);
    float v[VEC];
    if (r >= 0 && r < num_rows) {
      if constexpr (VEC == 1) {
        v[0] = to_float(src[r * row_stride + c * col_stride]);
      } else {
        VecIO<T, VEC>::load(src + r * row_stride + c, v);
      }
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] = 0.f;
    }
    VecIO<T, VEC>::store(dst + i * row_size + c, v);
  }
}

// One wave per (destination row, column block, slab).  DIRECT writes the row itself (one
// slab); otherwise fp32 partials (slab, row, col) go to scratch for the partials reduction.
template <typename T, typename I, int VEC, bool DIRECT>
__global__ __launch_bounds__(64) void scatter_rows_kernel(const I* __restrict__ indices, const T* __restrict__ values,
                                                          float* __restrict__ part, T* __restrict__ dst, int64_t n_idx,
                                                          int64_t num_rows, int64_t row_size, int64_t slab_len) {
  const int lane = threadIdx.x;
  const int64_t col = (static_cast<int64_t>(blockIdx.y) * 64 + lane) * VEC;
  const int64_t row = blockIdx.x;
  const int64_t slab = blockIdx.z;
  const int64_t i0 = slab * slab_len;
  const int64_t i1 = min(i0 + slab_len, n_idx);
  const bool active = col < row_size;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
  for (int64_t base = i0; base < i1; base += 64) {
    const int64_t mine = base + lane;
    const bool hit = mine < i1 && static_cast<int64_t>(indices[mine]) == row;
    uint64_t hits = __ballot(hit);
    while (hits) {  // wave-uniform: ascending index order
      const int bit = __ffsll(static_cast<long long>(hits)) - 1;
      hits &= hits - 1;
      if (active) {
        float v[VEC];
        VecIO<T, VEC>::load(values + (base + bit) * row_size + col, v);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += v[e];
      }
    }
  }
  if (!active) return;
  if constexpr (DIRECT) {
    VecIO<T, VEC>::store(dst + row * row_size + col, acc);
  } else {
    float* p = part + (slab * num_rows + row) * row_size + col;
#pragma unroll
    for (int e = 0; e < VEC; ++e) p[e] = acc[e];
  }
}

// ---- large tables: bucket the indices by destination row first ---------------------------

// key[i] = destination row of value row i (num_rows for an index outside the table: a bucket
// that nobody sums), pos[i] = i.
template <typename I>
__global__ __launch_bounds__(256) void scatter_keys_kernel(const I* __restrict__ indices, uint32_t* __restrict__ key,
                                                           uint32_t* __restrict__ pos, int64_t n_idx, int64_t num_rows) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n_idx) return;
  const int64_t r = static_cast<int64_t>(indices[i]);
  key[i] = static_cast<uint32_t>(r >= 0 && r < num_rows ? r : num_rows);
  pos[i] = static_cast<uint32_t>(i);
}

// ---- stable radix sort of (key, pos) pairs, eight bits of the key per pass --------------------
// A pass is three steps: the digit histogram of every tile of the list, an exclusive scan of
// the histograms in (digit, tile) order (per digit over the tiles, then over the digits'
// totals), and the scatter, in which a tile places its pairs behind its digit's offset in their
// order of appearance.  Counts are integer sums, so nothing
// depends on scheduling; equal keys keep their order in every pass, so after the last one the
// positions are ascending inside a key.

// hist[d * tiles + tile] = number of keys of the tile (256 * items consecutive pairs) with digit d
__global__ __launch_bounds__(256) void sort_hist_kernel(const uint32_t* __restrict__ key, uint32_t* __restrict__ hist,
                                                        int64_t n, int shift, int items, int tiles) {
  __shared__ uint32_t h[256];
  h[threadIdx.x] = 0;
  __syncthreads();
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * 256 * items;
  for (int e = 0; e < items; ++e) {
    const int64_t i = t0 + static_cast<int64_t>(e) * 256 + threadIdx.x;
    if (i < n) atomicAdd(&h[(key[i] >> shift) & 255u], 1u);
  }
  __syncthreads();
  hist[static_cast<int64_t>(threadIdx.x) * tiles + blockIdx.x] = h[threadIdx.x];
}

// Workgroup d turns digit d's row of counts, hist[d * tiles ..], into its exclusive scan over
// the tiles, 256 at a time, and leaves the digit's total in hist[256 * tiles + d].
__global__ __launch_bounds__(256) void sort_scan_kernel(uint32_t* __restrict__ hist, int tiles) {
  __shared__ uint32_t part[256];
  uint32_t* row = hist + static_cast<int64_t>(blockIdx.x) * tiles;
  uint32_t carry = 0;
  for (int t0 = 0; t0 < tiles; t0 += 256) {
    const int t = t0 + threadIdx.x;
    const uint32_t c = t < tiles ? row[t] : 0u;
    part[threadIdx.x] = c;
    __syncthreads();
    for (int d = 1; d < 256; d *= 2) {  // inclusive scan of the 256 counts
      const uint32_t v = threadIdx.x >= static_cast<unsigned>(d) ? part[threadIdx.x - d] : 0u;
      __syncthreads();
      part[threadIdx.x] += v;
      __syncthreads();
    }
    if (t < tiles) row[t] = carry + part[threadIdx.x] - c;
    carry += part[255];
    __syncthreads();
  }
  if (threadIdx.x == 0) hist[static_cast<int64_t>(256) * tiles + blockIdx.x] = carry;
}

// The pairs of a tile go behind hist[digit * tiles + tile], 256 at a time in their order: a
// pair's rank among the round's pairs with its digit is the number of lower lanes of its wave
// with that digit (eight ballots) plus the lower waves' counts of it.  The digit's offset is the
// total of the lower digits plus the digit's count in the tiles before; with RAW the histograms
// are still counts and every workgroup sums them itself (lists of few tiles: 256 * tiles reads
// a workgroup cost less than a launch of the scan).
template <bool RAW>
__global__ __launch_bounds__(256) void sort_scatter_kernel(const uint32_t* __restrict__ key, const uint32_t* __restrict__ pos,
                                                           uint32_t* __restrict__ key_out, uint32_t* __restrict__ pos_out,
                                                           const uint32_t* __restrict__ hist, int64_t n, int shift,
                                                           int items, int tiles) {
  __shared__ uint32_t base[256];
  __shared__ uint32_t wcount[4][256];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  {
    uint32_t total = 0, before = 0;  // of this thread's digit: in all tiles, in the tiles before this one
    if constexpr (RAW) {
      for (int t = 0; t < tiles; ++t) {
        const uint32_t c = hist[static_cast<int64_t>(threadIdx.x) * tiles + t];
        total += c;
        before += t < static_cast<int>(blockIdx.x) ? c : 0u;
      }
    } else {
      total = hist[static_cast<int64_t>(256) * tiles + threadIdx.x];
      before = hist[static_cast<int64_t>(threadIdx.x) * tiles + blockIdx.x];
    }
    uint32_t* scan = wcount[0];
    scan[threadIdx.x] = total;
    __syncthreads();
    for (int d = 1; d < 256; d *= 2) {
      const uint32_t v = threadIdx.x >= static_cast<unsigned>(d) ? scan[threadIdx.x - d] : 0u;
      __syncthreads();
      scan[threadIdx.x] += v;
      __syncthreads();
    }
    base[threadIdx.x] = scan[threadIdx.x] - total + before;
    __syncthreads();
  }
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * 256 * items;
  for (int e = 0; e < items; ++e) {
#pragma unroll
    for (int w = 0; w < 4; ++w) wcount[w][threadIdx.x] = 0;
    __syncthreads();
    const int64_t i = t0 + static_cast<int64_t>(e) * 256 + threadIdx.x;
    const bool valid = i < n;
    const uint32_t k = valid ? key[i] : 0u;
    const uint32_t d = (k >> shift) & 255u;
    uint64_t same = __ballot(valid);
#pragma unroll
    for (int bit = 0; bit < 8; ++bit) {
      const bool one = (d >> bit) & 1u;
      const uint64_t m = __ballot(one);
      same &= one ? m : ~m;
    }
    const uint32_t below = static_cast<uint32_t>(__popcll(same & ((uint64_t{1} << lane) - 1)));
    if (valid && below == 0) wcount[wave][d] = static_cast<uint32_t>(__popcll(same));
    __syncthreads();
    if (valid) {
      uint32_t r = base[d] + below;
      for (int w = 0; w < wave; ++w) r += wcount[w][d];
      key_out[r] = k;
      pos_out[r] = pos[i];
    }
    __syncthreads();
    base[threadIdx.x] += wcount[0][threadIdx.x] + wcount[1][threadIdx.x] + wcount[2][threadIdx.x] + wcount[3][threadIdx.x];
    __syncthreads();
  }
}

// Runs of equal keys in the sorted list: row k's value rows are pos[first[k] .. last[k]).
// `first` and `last` hold zeros on entry, so a row without values gets an empty run.
__global__ __launch_bounds__(256) void scatter_runs_kernel(const uint32_t* __restrict__ key, uint32_t* __restrict__ first,
                                                           uint32_t* __restrict__ last, int64_t n_idx) {
  const int64_t p = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (p >= n_idx) return;
  const uint32_t k = key[p];
  if (p == 0 || key[p - 1] != k) first[k] = static_cast<uint32_t>(p);
  if (p == n_idx - 1 || key[p + 1] != k) last[k] = static_cast<uint32_t>(p + 1);
}

// One wave per (destination row, column block): the row's value rows added in ascending
// position order in fp32 (the order of scatter_rows_kernel with one slab, so the two agree
// bit for bit); rows without values are written as zeros.
template <typename T, int VEC>
__global__ __launch_bounds__(64) void scatter_runs_sum_kernel(const uint32_t* __restrict__ pos,
                                                              const uint32_t* __restrict__ first,
                                                              const uint32_t* __restrict__ last,
                                                              const T* __restrict__ values, T* __restrict__ dst,
                                                              int64_t row_size) {
  const int64_t col = (static_cast<int64_t>(blockIdx.y) * 64 + threadIdx.x) * VEC;
  const int64_t row = blockIdx.x;
  if (col >= row_size) return;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
  const uint32_t p1 = last[row];
  for (uint32_t p = first[row]; p < p1; ++p) {
    float v[VEC];
    VecIO<T, VEC>::load(values + static_cast<int64_t>(pos[p]) * row_size + col, v);
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] += v[e];
  }
  VecIO<T, VEC>::store(dst + row * row_size + col, acc);
}

template <typename T, typename I, int VEC>
static int scatter_bucketed(const I* indices, const T* values, T* dst, int64_t n_idx, int64_t num_rows, int64_t row_size,
                            hipStream_t s) {
  int bits = 1;
  while (bits < 32 && (int64_t{1} << bits) <= num_rows) ++bits;  // keys are 0 .. num_rows
  const int passes = (bits + 7) / 8;
  // tiles of 256 * items pairs: four pairs per thread while that fills the chip, more for long
  // lists (a tile's pairs of one digit land next to each other, and every tile costs 256
  // counters); MOGRAD_HIP_SCATTER_SORT_MAX_TILES moves the limit
  const int64_t max_tiles = std::max(1, env_int("MOGRAD_HIP_SCATTER_SORT_MAX_TILES", 1024));
  const int items = static_cast<int>(std::max<int64_t>(4, ceil_div(n_idx, 256 * max_tiles)));
  const int tiles = static_cast<int>(ceil_div(n_idx, int64_t{256} * items));
  // one block: key, pos, their second copies (n each), first, last (num_rows + 1 each), the histograms
  const int64_t ints = 4 * n_idx + 2 * (num_rows + 1) + int64_t{256} * (tiles + 1);
  Scratch work;
  MG_TRY(work.take(ints * 4));
  uint32_t* key = work.as<uint32_t>();
  uint32_t* pos = key + n_idx;
  uint32_t* key2 = pos + n_idx;
  uint32_t* pos2 = key2 + n_idx;
  uint32_t* first = pos2 + n_idx;
  uint32_t* last = first + num_rows + 1;
  uint32_t* hist = last + num_rows + 1;
  const unsigned blocks = static_cast<unsigned>(ceil_div(n_idx, 256));
  MG_TRY(mg_fill(first, 0.0, 2 * (num_rows + 1), MG_I32, s));
  hipLaunchKernelGGL((scatter_keys_kernel<I>), dim3(blocks), dim3(256), 0, s, indices, key, pos, n_idx, num_rows);
  MG_LAUNCH_CHECK();
  for (int p = 0; p < passes; ++p) {
    hipLaunchKernelGGL(sort_hist_kernel, dim3(tiles), dim3(256), 0, s, key, hist, n_idx, 8 * p, items, tiles);
    if (tiles <= 64) {
      hipLaunchKernelGGL(sort_scatter_kernel<true>, dim3(tiles), dim3(256), 0, s, key, pos, key2, pos2, hist, n_idx, 8 * p,
                         items, tiles);
    } else {
      hipLaunchKernelGGL(sort_scan_kernel, dim3(256), dim3(256), 0, s, hist, tiles);
      hipLaunchKernelGGL(sort_scatter_kernel<false>, dim3(tiles), dim3(256), 0, s, key, pos, key2, pos2, hist, n_idx, 8 * p,
                         items, tiles);
    }
    MG_LAUNCH_CHECK();
    std::swap(key, key2);
    std::swap(pos, pos2);
  }
  uint32_t* key_sorted = key;
  uint32_t* pos_sorted = pos;
  hipLaunchKernelGGL(scatter_runs_kernel, dim3(blocks), dim3(256), 0, s, key_sorted, first, last, n_idx);
  MG_LAUNCH_CHECK();
  const dim3 grid(static_cast<unsigned>(num_rows), static_cast<unsigned>(ceil_div(row_size, 64 * VEC)));
  hipLaunchKernelGGL((scatter_runs_sum_kernel<T, VEC>), grid, dim3(64), 0, s, pos_sorted, first, last, values, dst, row_size);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T, typename I>
static int gather_typed(const void* src, const void* indices, void* dst, int64_t n_idx, int64_t num_rows,
                        int64_t row_size, int64_t row_stride, int64_t col_stride, hipStream_t s) {
  constexpr int WIDE = WideVec<T>::value;
  const bool wide = col_stride == 1 && row_size % WIDE == 0 && row_stride % WIDE == 0 && aligned16(src) && aligned16(dst);
  const int64_t chunks = n_idx * (wide ? row_size / WIDE : row_size);
  int64_t blocks = ceil_div(chunks, 256);
  const int64_t cap = static_cast<int64_t>(device_info().cu_count) * 16;
  if (blocks > cap) blocks = cap;
  const dim3 grid(static_cast<unsigned>(blocks));
  if (wide)
    hipLaunchKernelGGL((gather_rows_kernel<T, I, WIDE>), grid, dim3(256), 0, s, static_cast<const T*>(src),
                       static_cast<const I*>(indices), static_cast<T*>(dst), n_idx, num_rows, row_size, row_stride,
                       col_stride);
  else
    hipLaunchKernelGGL((gather_rows_kernel<T, I, 1>), grid, dim3(256), 0, s, static_cast<const T*>(src),
                       static_cast<const I*>(indices), static_cast<T*>(dst), n_idx, num_rows, row_size, row_stride,
                       col_stride);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T, typename I, int VEC>
static int scatter_launch(const I* indices, const T* values, T* dst, int64_t n_idx, int64_t num_rows, int64_t row_size,
                          hipStream_t s) {
  // Tables of a thousand rows and more: bucket first (MOGRAD_HIP_SCATTER_BUCKET_MIN_ROWS moves
  // the threshold; (50304, 768) from 8192 rows took 5 ms by scanning).
  if (num_rows >= env_int("MOGRAD_HIP_SCATTER_BUCKET_MIN_ROWS", 1024) && n_idx > 0 && n_idx < 0x7fffffffLL &&
      num_rows < 0x7fffffffLL)
    return scatter_bucketed<T, I, VEC>(indices, values, dst, n_idx, num_rows, row_size, s);
  const int64_t col_blocks = ceil_div(row_size, 64 * VEC);
  // Slabs of the index list: enough waves to fill the device, at least 256 indices each,
  // partial sums capped at 64 MiB.
  int64_t slabs = ceil_div(static_cast<int64_t>(device_info().cu_count) * 16, num_rows * col_blocks);
  const int64_t by_len = ceil_div(n_idx, 256);
  if (slabs > by_len) slabs = by_len;
  const int64_t by_bytes = (int64_t{64} << 20) / (num_rows * row_size * static_cast<int64_t>(sizeof(float)));
  if (slabs > by_bytes) slabs = by_bytes;
  if (slabs > 65535) slabs = 65535;
  if (slabs < 1) slabs = 1;
  const int64_t slab_len = ceil_div(ceil_div(n_idx, slabs), 64) * 64;
  slabs = n_idx > 0 ? ceil_div(n_idx, slab_len) : 1;
  const dim3 grid(static_cast<unsigned>(num_rows), static_cast<unsigned>(col_blocks), static_cast<unsigned>(slabs));
  if (slabs == 1) {
    hipLaunchKernelGGL((scatter_rows_kernel<T, I, VEC, true>), grid, dim3(64), 0, s, indices, values, nullptr, dst,
                       n_idx, num_rows, row_size, slab_len);
    MG_LAUNCH_CHECK();
    return MG_OK;
  }
  Scratch part;
  MG_TRY(part.take(slabs * num_rows * row_size * static_cast<int64_t>(sizeof(float))));
  hipLaunchKernelGGL((scatter_rows_kernel<T, I, VEC, false>), grid, dim3(64), 0, s, indices, values, part.as<float>(),
                     dst, n_idx, num_rows, row_size, slab_len);
  MG_LAUNCH_CHECK();
  const int64_t cols = num_rows * row_size;
  reduce_partials_or_defer<T>(part, dst, nullptr, static_cast<T*>(nullptr), slabs, cols, device_info().cu_count, s);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T, typename I>
static int scatter_typed(const void* indices, const void* values, void* dst, int64_t n_idx, int64_t num_rows,
                         int64_t row_size, hipStream_t s) {
  constexpr int WIDE = WideVec<T>::value;
  const bool wide = row_size % WIDE == 0 && aligned16(values) && aligned16(dst);
  if (wide)
    return scatter_launch<T, I, WIDE>(static_cast<const I*>(indices), static_cast<const T*>(values),
                                      static_cast<T*>(dst), n_idx, num_rows, row_size, s);
  return scatter_launch<T, I, 1>(static_cast<const I*>(indices), static_cast<const T*>(values), static_cast<T*>(dst),
                                 n_idx, num_rows, row_size, s);
}

template <typename T>
static int gather_by_index(const void* src, const void* indices, void* dst, int64_t n_idx, int64_t num_rows,
                           int64_t row_size, int64_t row_stride, int64_t col_stride, int idx_dtype, hipStream_t s) {
  if (idx_dtype == MG_I32)
    return gather_typed<T, int32_t>(src, indices, dst, n_idx, num_rows, row_size, row_stride, col_stride, s);
  return gather_typed<T, int64_t>(src, indices, dst, n_idx, num_rows, row_size, row_stride, col_stride, s);
}

template <typename T>
static int scatter_by_index(const void* indices, const void* values, void* dst, int64_t n_idx, int64_t num_rows,
                            int64_t row_size, int idx_dtype, hipStream_t s) {
  if (idx_dtype == MG_I32) return scatter_typed<T, int32_t>(indices, values, dst, n_idx, num_rows, row_size, s);
  return scatter_typed<T, int64_t>(indices, values, dst, n_idx, num_rows, row_size, s);
}

}  // namespace mg

extern "C" {

int mg_gather(const void* src, const void* indices, void* dst, int64_t n_idx, int64_t num_rows, int64_t row_size,
              int64_t src_row_stride, int64_t src_col_stride, int idx_dtype, int dtype, mg_stream stream) {
  if (!mg::is_float_dtype(dtype)) return mg::fail(MG_ERR_INVALID, "gather: unsupported dtype %s", mg::dtype_name(dtype));
  if (idx_dtype != MG_I32 && idx_dtype != MG_I64)
    return mg::fail(MG_ERR_INVALID, "gather: indices must be int32 or int64, got %s", mg::dtype_name(idx_dtype));
  if (n_idx < 0 || num_rows < 0 || row_size < 0 || src_row_stride < 0 || src_col_stride < 0)
    return mg::fail(MG_ERR_INVALID, "gather: negative size or stride");
  if (n_idx == 0 || row_size == 0) return MG_OK;
  if (!indices || !dst || (num_rows > 0 && !src)) return mg::fail(MG_ERR_INVALID, "gather: null pointer argument");
  hipStream_t s = mg::to_stream(stream);
  switch (dtype) {
    case MG_F32:
      return mg::gather_by_index<float>(src, indices, dst, n_idx, num_rows, row_size, src_row_stride, src_col_stride,
                                        idx_dtype, s);
    case MG_F16:
      return mg::gather_by_index<mg::f16_t>(src, indices, dst, n_idx, num_rows, row_size, src_row_stride,
                                            src_col_stride, idx_dtype, s);
    default:
      return mg::gather_by_index<mg::bf16_t>(src, indices, dst, n_idx, num_rows, row_size, src_row_stride,
                                             src_col_stride, idx_dtype, s);
  }
}

int mg_scatter_add_deferred(const void* indices, const void* values, void* dst, int64_t n_idx, int64_t num_rows,
                            int64_t row_size, int idx_dtype, int dtype, int grad_dtype, mg_deferred list,
                            mg_stream stream) {
  if (!mg::is_float_dtype(dtype))
    return mg::fail(MG_ERR_INVALID, "scatter_add_deferred: unsupported dtype %s", mg::dtype_name(dtype));
  MG_TRY(mg::deferred_check("scatter_add_deferred", list, dtype, grad_dtype));
  if (num_rows < 0 || row_size < 0) return mg::fail(MG_ERR_INVALID, "scatter_add_deferred: negative size");
  mg::DeferredScope scope(static_cast<mg::DeferredList*>(list), dtype, grad_dtype);
  void* dst_use;
  MG_TRY(scope.substitute(dst, num_rows * row_size, &dst_use));
  MG_TRY(mg_scatter_add(indices, values, dst_use, n_idx, num_rows, row_size, idx_dtype, dtype, stream));
  return scope.finish(mg::to_stream(stream));
}

int mg_scatter_add(const void* indices, const void* values, void* dst, int64_t n_idx, int64_t num_rows,
                   int64_t row_size, int idx_dtype, int dtype, mg_stream stream) {
  if (!mg::is_float_dtype(dtype))
    return mg::fail(MG_ERR_INVALID, "scatter_add: unsupported dtype %s", mg::dtype_name(dtype));
  if (idx_dtype != MG_I32 && idx_dtype != MG_I64)
    return mg::fail(MG_ERR_INVALID, "scatter_add: indices must be int32 or int64, got %s", mg::dtype_name(idx_dtype));
  if (n_idx < 0 || num_rows < 0 || row_size < 0) return mg::fail(MG_ERR_INVALID, "scatter_add: negative size");
  if (num_rows == 0 || row_size == 0) return MG_OK;
  if (num_rows > INT32_MAX || row_size > int64_t{65535} * 64)
    return mg::fail(MG_ERR_UNSUPPORTED, "scatter_add: destination (%lld, %lld) exceeds the launch grid",
                    static_cast<long long>(num_rows), static_cast<long long>(row_size));
  if (!dst || (n_idx > 0 && (!indices || !values))) return mg::fail(MG_ERR_INVALID, "scatter_add: null pointer argument");
  hipStream_t s = mg::to_stream(stream);
  switch (dtype) {
    case MG_F32: return mg::scatter_by_index<float>(indices, values, dst, n_idx, num_rows, row_size, idx_dtype, s);
    case MG_F16: return mg::scatter_by_index<mg::f16_t>(indices, values, dst, n_idx, num_rows, row_size, idx_dtype, s);
    default: return mg::scatter_by_index<mg::bf16_t>(indices, values, dst, n_idx, num_rows, row_size, idx_dtype, s);
  }
}

}  // extern "C"
