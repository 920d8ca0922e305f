// Row gather (embedding lookup) and its gradient, the row scatter-add.
//
// The scatter-add uses no atomics: each wave owns one destination row (and one slab of
// the index list), scans the indices 64 at a time, and adds the matching value rows in
// index order with fp32 accumulation, so the result does not depend on scheduling.
// That costs rows x indices comparisons, fine for a 65-row table and hopeless for a 50304-row
// one; large tables first sort (row, position) pairs by row (a stable radix sort, so
// positions stay ascending inside a row), and a wave then adds only its own row's run.
#include <algorithm>
#include <atomic>
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

// VEC elements of a value row as loaded, unpacked to floats only when they are added: eight
// of them wait in registers for the loads of a long run.
template <typename T, int VEC>
struct PackedChunk {
  static constexpr int kBytes = sizeof(T) * VEC;
  static_assert(kBytes == 16 || kBytes == 4 || kBytes == 2, "a chunk is one 16-byte load or one element");
  uint32_t w[kBytes == 16 ? 4 : 1];
  __device__ __forceinline__ void load(const T* p) {
    if constexpr (kBytes == 16) {
      const mg_u4 r = *reinterpret_cast<const mg_u4*>(p);
      w[0] = r[0]; w[1] = r[1]; w[2] = r[2]; w[3] = r[3];
    } else if constexpr (kBytes == 4) {
      w[0] = *reinterpret_cast<const uint32_t*>(p);
    } else {
      w[0] = *reinterpret_cast<const uint16_t*>(p);
    }
  }
  __device__ __forceinline__ void unpack(float (&v)[VEC]) {
#pragma unroll
    for (int i = 0; i < (kBytes == 16 ? 4 : 1); ++i) asm volatile("" : "+v"(w[i]));  // not before this point
    if constexpr (kBytes == 2) {
      const uint16_t bits = static_cast<uint16_t>(w[0]);
      T t;
      __builtin_memcpy(&t, &bits, 2);
      v[0] = to_float(t);
    } else {
      VecIO<T, VEC>::load(reinterpret_cast<const T*>(w), v);
    }
  }
};

// ---- large tables, short index lists: one launch ------------------------------------------
// A workgroup owns 4 * rows_per_wave consecutive destination rows and one block of 64 * VEC
// columns.  Its four waves read a quarter of the index list each and keep, in position order,
// the (row, position) pairs that fall into the workgroup's rows; the four lists one after the
// other are then the workgroup's pairs in position order.  After that a wave walks the lists
// once per row of its own and adds the value rows it finds, in that order, in fp32 from zero
// (the order of scatter_rows_kernel with one slab: the same bits), and writes the row, zeros if
// it found none.  Every workgroup reads the whole index list, which is what limits this form
// to short lists; it needs no sort and no second launch.
constexpr int kRangeCap = 512;      // pairs of a wave's list kept in LDS
constexpr int kRangePosBits = 25;   // a pair is (row - first row) << 25 | position
constexpr uint32_t kRangePosMask = (1u << kRangePosBits) - 1;

// The pairs of positions [i0, i1) with a row in [r0, r1), written to out[0 .. cap) in position
// order; returns their number, which may exceed cap (the pairs beyond it are then not kept).
// A lane reads 16 bytes of indices at once where it can.
template <typename I>
__device__ __forceinline__ uint32_t range_collect(const I* __restrict__ indices, int64_t i0, int64_t i1, int64_t r0, int64_t r1,
                                                  uint32_t* out, uint32_t cap, bool vec_ok, int lane) {
  constexpr int K = 16 / sizeof(I);
  constexpr int U = 4;  // loads in flight
  struct alignas(16) Pack {
    I v[K];
  };
  const uint64_t lower = (uint64_t{1} << lane) - 1;
  uint32_t cnt = 0;
  for (int64_t base = i0; base < i1; base += 64 * K * U) {
    Pack pk[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t p = base + (u * 64 + lane) * K;
      if (vec_ok && p + K <= i1) {
        pk[u] = *reinterpret_cast<const Pack*>(indices + p);
      } else {
#pragma unroll
        for (int c = 0; c < K; ++c) pk[u].v[c] = p + c < i1 ? indices[p + c] : static_cast<I>(-1);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t p = base + (u * 64 + lane) * K;
      bool hit[K];
      uint64_t found[K], any = 0;
#pragma unroll
      for (int c = 0; c < K; ++c) {
        const int64_t v = static_cast<int64_t>(pk[u].v[c]);
        hit[c] = v >= r0 && v < r1;
        found[c] = __ballot(hit[c]);
        any |= found[c];
      }
      if (any) {  // wave-uniform; a lane's pairs follow those of the lower lanes
        uint32_t slot = cnt;
#pragma unroll
        for (int c = 0; c < K; ++c) {
          slot += static_cast<uint32_t>(__popcll(found[c] & lower));
          cnt += static_cast<uint32_t>(__popcll(found[c]));
        }
#pragma unroll
        for (int c = 0; c < K; ++c) {
          if (hit[c]) {
            if (slot < cap)
              out[slot] = (static_cast<uint32_t>(static_cast<int64_t>(pk[u].v[c]) - r0) << kRangePosBits) |
                          static_cast<uint32_t>(p + c);
            ++slot;
          }
        }
      }
    }
  }
  return cnt;
}

// grid (row ranges, column blocks).  `quarter` is the share of the index list a wave reads, a
// multiple of 256.  A workgroup whose lists outgrow LDS (a row that a large part of the list
// points at) keeps them in one of the `slots` areas of 4 * quarter pairs behind the `slots`
// owner words at `spill`: it claims an area by writing `tag`, a number no earlier launch on
// this memory has used, over an owner word that does not hold it yet, so the words need no
// clearing, and which area it gets does not change what it computes.  More than
// n_idx / (kRangeCap + 1) workgroups per column block cannot outgrow LDS, so with that many
// areas a free one is always found; a workgroup that finds none (fewer areas, or stale words
// that happen to equal the tag) reads the whole index list once per row instead.
template <typename T, typename I, int VEC, bool STREAM>
__global__ __launch_bounds__(256) void scatter_ranges_kernel(const I* __restrict__ indices, const T* __restrict__ values,
                                                             T* __restrict__ dst, uint32_t* __restrict__ spill, uint32_t slots,
                                                             uint32_t tag, int64_t n_idx, int64_t num_rows, int64_t row_size,
                                                             int rows_per_wave, int64_t quarter, bool vec_ok) {
  __shared__ uint32_t lds_list[4 * kRangeCap];
  __shared__ uint32_t counts[4];
  __shared__ int claimed;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * 4 * rows_per_wave;
  const int64_t r1 = min(r0 + 4 * rows_per_wave, num_rows);
  const int64_t i0 = min(wave * quarter, n_idx), i1 = min(i0 + quarter, n_idx);
  {
    const uint32_t cnt = range_collect<I>(indices, i0, i1, r0, r1, lds_list + wave * kRangeCap, kRangeCap, vec_ok, lane);
    if (lane == 0) counts[wave] = cnt;
  }
  __syncthreads();
  const uint32_t c0 = counts[0], c1 = counts[1], c2 = counts[2], c3 = counts[3];
  const uint32_t* list = lds_list;  // LDS or global memory
  int64_t stride = kRangeCap;
  const int64_t col = (static_cast<int64_t>(blockIdx.y) * 64 + lane) * VEC;
  const bool active = col < row_size;
  const uint32_t col32 = static_cast<uint32_t>(col);  // a row holds fewer than 2^22 columns
  auto put = [&](int64_t row, const float (&acc)[VEC]) {
    if constexpr (STREAM) VecIO<T, VEC>::store_stream(dst + row * row_size + col, acc);
    else VecIO<T, VEC>::store(dst + row * row_size + col, acc);
  };
  if (max(max(c0, c1), max(c2, c3)) > kRangeCap) {  // the same for the whole workgroup
    if (threadIdx.x == 0) {
      int got = -1;
      uint32_t at = slots ? (blockIdx.y * gridDim.x + blockIdx.x) % slots : 0;
      for (uint32_t tries = 0; tries < slots && got < 0; ++tries) {
        uint32_t seen = __hip_atomic_load(spill + at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        while (seen != tag) {  // free: claim it unless another workgroup does first
          const uint32_t before = atomicCAS(spill + at, seen, tag);
          if (before == seen) {
            got = static_cast<int>(at);
            break;
          }
          seen = before;
        }
        at = at + 1 == slots ? 0 : at + 1;
      }
      claimed = got;
    }
    __syncthreads();
    if (claimed < 0) {  // no area: a wave reads the whole list for each row of its own
      for (int k = 0; k < rows_per_wave; ++k) {
        const int64_t row = r0 + wave * rows_per_wave + k;
        if (row >= r1) break;
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
        for (int64_t base = 0; base < n_idx; base += 64) {
          const int64_t at = base + lane;
          uint64_t hits = __ballot(at < n_idx && static_cast<int64_t>(indices[at]) == row);
          while (hits) {
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
        if (active) put(row, acc);
      }
      return;
    }
    uint32_t* mine = spill + slots + static_cast<int64_t>(claimed) * 4 * quarter;
    range_collect<I>(indices, i0, i1, r0, r1, mine + wave * quarter, static_cast<uint32_t>(quarter), vec_ok, lane);
    __threadfence();
    __syncthreads();
    list = mine;
    stride = quarter;
  }
  const uint32_t off1 = c0, off2 = off1 + c1, off3 = off2 + c2, total = off3 + c3;
  auto pair_at = [&](uint32_t t) -> uint32_t {  // the t-th pair of the four lists in a row
    if (t >= total) return 0xffffffffu;          // row field 127: no row of the workgroup
    const int l = (t >= off1) + (t >= off2) + (t >= off3);
    const uint32_t first = l == 0 ? 0u : (l == 1 ? off1 : (l == 2 ? off2 : off3));
    return list[l * stride + (t - first)];
  };
  const uint32_t head = pair_at(lane);  // most workgroups hold fewer than 64 pairs
  for (int k = 0; k < rows_per_wave; ++k) {
    const uint32_t local = static_cast<uint32_t>(wave * rows_per_wave + k);
    const int64_t row = r0 + local;
    if (row >= r1) break;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
    for (uint32_t b = 0; b < total; b += 64) {
      const uint32_t pair = b == 0 ? head : pair_at(b + lane);
      uint64_t hits = __ballot((pair >> kRangePosBits) == local);
      while (hits) {  // wave-uniform; eight value rows in flight, added in position order
        constexpr int U = 8;
        uint32_t pos[U];
        int got = 0;
#pragma unroll
        for (int u = 0; u < U; ++u) {
          pos[u] = 0;
          if (hits) {
            const int bit = __ffsll(static_cast<long long>(hits)) - 1;
            hits &= hits - 1;
            pos[u] = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(pair), bit)) & kRangePosMask;
            got = u + 1;
          }
        }
        if (active) {
          PackedChunk<T, VEC> chunk[U];
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (u < got) chunk[u].load(values + static_cast<int64_t>(pos[u]) * row_size + col32);
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (u < got) {
              float v[VEC];
              chunk[u].unpack(v);
#pragma unroll
              for (int e = 0; e < VEC; ++e) acc[e] += v[e];
            }
        }
      }
    }
    if (active) put(row, acc);
  }
}

// One count for every instantiation below: a tag must differ from those of all earlier launches
// that may have used the same pool block.
static std::atomic<uint32_t> g_range_launches{0};

template <typename T, typename I, int VEC>
static int scatter_ranges(const I* indices, const T* values, T* dst, int64_t n_idx, int64_t num_rows, int64_t row_size,
                          int rows_per_wave, int64_t quarter, hipStream_t s) {
  const int64_t ranges = ceil_div(num_rows, 4 * rows_per_wave), col_blocks = ceil_div(row_size, 64 * VEC);
  const uint32_t tag = ++g_range_launches;
  // as many areas as workgroups can need, within 64 MiB
  int64_t slots = std::min(col_blocks * (n_idx / (kRangeCap + 1) + 1) + 8, std::max<int64_t>(1, (int64_t{4} << 20) / quarter));
  const int slots_knob = env_int("MOGRAD_HIP_SCATTER_SPILL_SLOTS", -1);  // tests: 0 = no areas
  if (slots_knob >= 0) slots = slots_knob;
  Scratch spill;
  MG_TRY(spill.take((slots + slots * 4 * quarter + 1) * 4));
  const dim3 grid(static_cast<unsigned>(ranges), static_cast<unsigned>(col_blocks));
  const bool stream_out = env_int("MOGRAD_HIP_SCATTER_STREAM", 1) != 0;
  auto kernel = stream_out ? scatter_ranges_kernel<T, I, VEC, true> : scatter_ranges_kernel<T, I, VEC, false>;
  hipLaunchKernelGGL(kernel, grid, dim3(256), 0, s, indices, values, dst, spill.as<uint32_t>(), static_cast<uint32_t>(slots), tag, n_idx,
                     num_rows, row_size, rows_per_wave, quarter, aligned16(indices));
  MG_LAUNCH_CHECK();
  return MG_OK;
}

// ---- large tables, long index lists: bucket the indices by destination row first -------------

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
  const uint32_t col32 = static_cast<uint32_t>(col);
  const uint32_t p1 = last[row];
  for (uint32_t p = first[row]; p < p1; p += 8) {  // eight value rows in flight
    const int got = static_cast<int>(min(p1 - p, 8u));
    PackedChunk<T, VEC> chunk[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (u < got) chunk[u].load(values + static_cast<int64_t>(pos[p + u]) * row_size + col32);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (u < got) {
        float v[VEC];
        chunk[u].unpack(v);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += v[e];
      }
  }
  VecIO<T, VEC>::store_stream(dst + row * row_size + col, acc);
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
      num_rows < 0x7fffffffLL) {
    // Short lists: every workgroup of a row range reads the whole list, up to 2^(the knob)
    // index reads in all (MOGRAD_HIP_SCATTER_RANGE_READS_LOG2; 0 switches the form off), and a
    // wave's list should hold 128 pairs at most when the indices are spread evenly.
    const int rows_per_wave = static_cast<int>(std::min<int64_t>(16, std::max<int64_t>(1, num_rows / 4096)));
    constexpr int64_t kStep = 64 * (16 / sizeof(I)) * 4;  // positions a wave reads in one step
    const int64_t quarter = ceil_div(ceil_div(n_idx, 4), kStep) * kStep;
    const int64_t reads = ceil_div(num_rows, 4 * rows_per_wave) * ceil_div(row_size, 64 * VEC) * 4 * quarter;
    const int reads_log2 = env_int("MOGRAD_HIP_SCATTER_RANGE_READS_LOG2", 27);
    if (reads_log2 > 0 && reads_log2 < 40 && reads <= (int64_t{1} << reads_log2) && n_idx < (int64_t{1} << kRangePosBits) &&
        n_idx * rows_per_wave <= 128 * num_rows)
      return scatter_ranges<T, I, VEC>(indices, values, dst, n_idx, num_rows, row_size, rows_per_wave, quarter, s);
    return scatter_bucketed<T, I, VEC>(indices, values, dst, n_idx, num_rows, row_size, s);
  }
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
