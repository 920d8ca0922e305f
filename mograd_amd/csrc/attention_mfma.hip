// Flash attention on the matrix cores for 16-bit storage (bf16, fp16), head dim <= 128.
//
// All three kernels use v_mfma_f32_32x32x16 with fp32 accumulation and share one idea:
// the tensor that a workgroup keeps for its whole life sits in registers as the MFMA's
// B operand (column = lane), the tensor that streams past comes through LDS as the A
// operand, and the 32x32 score tile comes out with "column = lane, rows in runs of four",
// which is exactly the B-operand shape of the next product, so probabilities and score
// gradients never leave registers.
//
//   forward   workgroup = 128 queries (4 waves x 32); streams 64-key blocks.
//             S^T = K Q^T, online softmax per lane (lane = one query), O^T += V^T P^T.
//   dQ        same shape; S^T and dP^T = V dO^T, dS^T = P (dP - delta), dQ^T += K^T dS^T.
//   dK, dV    workgroup = 128 keys (4 waves x 32); streams 64-query blocks.
//             S = Q K^T, dP = dO V^T, dV^T += dO^T P, dK^T += Q^T dS.
// dQ has its own kernel that recomputes S and dP: seven products instead of five, but no
// atomics, so every output is written once and results are reproducible.
//
// A product that contracts over the streamed index needs the streamed tile transposed
// ([d][row]).  A tile is staged in LDS once, row-major with its 16-byte chunks swizzled; the
// products that contract over its columns read it with ds_read_b128, the ones that contract
// over its rows with ds_read_b64_tr_b16, which transposes 4 x 16 blocks on the way out.
// For head dims up to 64 without a bias the backward walks are software-pipelined
// (attn_dkdv_pipe_block, attn_dq_pipe_block): tiles copied global -> LDS by
// global_load_lds_dwordx4 into a ring of three buffers, the exponentials of one tile issued
// between the matrix instructions of its neighbours.
//
// Layouts: Q, K, V, dQ, dK, dV BSHD; O, dO BHSD; mask (B,H,S,S); LSE, delta (B,H,S) fp32.
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "attention_generic.h"
#include "mg_internal.h"

namespace mg {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

template <typename T>
struct Mma;
template <>
struct Mma<bf16_t> {
  static __device__ __forceinline__ floatx16 run(uint4 a, uint4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0,
                                                   0, 0);
  }
  // Two fp32 -> packed pair, round to nearest even (one v_cvt_pk_bf16_f32).
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    const float2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  }
  static __device__ __forceinline__ float2_t unpack2(uint32_t w) {
    return __builtin_convertvector(__builtin_bit_cast(bf16x2_t, w), float2_t);
  }
};
template <>
struct Mma<f16_t> {
  static __device__ __forceinline__ floatx16 run(uint4 a, uint4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0,
                                                  0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    const float2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
  }
  static __device__ __forceinline__ float2_t unpack2(uint32_t w) {
    return __builtin_convertvector(__builtin_bit_cast(f16x2_t, w), float2_t);
  }
};

// Eight packed elements times `f`, rounded back to T.  Used once per workgroup to fold the
// softmax scale (times log2 e) into the resident operand of the score product, so that the
// product comes out of the matrix core already in the exponent's units.
template <typename T>
__device__ __forceinline__ uint4 scale_frag(uint4 v, float f) {
  const uint32_t in[4] = {v.x, v.y, v.z, v.w};
  uint32_t out[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float2_t x = Mma<T>::unpack2(in[i]);
    out[i] = Mma<T>::pack2(x[0] * f, x[1] * f);
  }
  return make_uint4(out[0], out[1], out[2], out[3]);
}

// Makes a fragment loaded from global memory before a loop count as "arrived" at this
// point.  Without it the compiler's wait-count bookkeeping treats the load as possibly
// still in flight at the loop header and waits for *all* outstanding global loads at the
// fragment's first use inside the loop, which also drains the tile prefetch issued a few
// instructions earlier.
__device__ __forceinline__ void settle(uint4& v) { asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w)); }

__device__ __forceinline__ floatx16 splat16(float v) {
  floatx16 z;
#pragma unroll
  for (int r = 0; r < 16; ++r) z[r] = v;
  return z;
}

constexpr int kAttnThreads = 256;
typedef short short4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float fexp2(float v) { return __builtin_amdgcn_exp2f(v); }

// ---- LDS tiles -------------------------------------------------------------------------
// A staged tile is R rows x DP columns of T, row-major, rows of DP * 2 bytes without padding.
// The 16-byte chunk c of row r is stored at chunk position c ^ swz(r) (low three bits), with
// swz(r) = 2 * (r % 4) + (r / 4) % 2.  The transposing 64-bit reads (16 lanes: four rows x 32
// bytes) and the staging stores are free of bank conflicts with it; the 128-bit row reads
// are served two rows per bank group (LDS has 64 banks and serves 16 lanes of a 128-bit
// read per clock; timed with four waves reading back to back: 32 clocks per read against
// 19 for consecutive addresses).  A swizzle over r % 16 that removes that too, 4 * (r/2 % 2)
// + (r/4 % 4), was measured in these kernels: 25 % fewer LDS-busy cycles, but the two
// transposing reads of a fragment then need separate address registers and adds, and the
// forward, which is bound by its VALU work, ran 3-5 % slower (backward within 1 %).  Storing
// tile row r in LDS row (r & ~15) | r3 | r0 << 1 | r1 << 2 | r2 << 3 instead keeps this swizzle,
// spreads the row reads over all banks and leaves the second transposing read at a constant
// distance; it measured the same as this layout to within 2 % either way (forward at
// S = 4096 4 % slower, D = 128 backward 2 % faster).  LDS conflicts are not what limits
// these kernels, so the plain row order stays.  One image serves the products that contract over the tile's columns and
// those that contract over its rows.
template <int DP>
constexpr int tile_row_bytes() { return DP * 2; }
__device__ __forceinline__ int tile_swz(int r) { return 2 * (r % 4) + (r / 4) % 2; }
template <int DP>
__device__ __forceinline__ int tile_chunk_at(int r, int c) { return r * tile_row_bytes<DP>() + ((c ^ tile_swz(r)) * 16); }

// Global -> registers -> LDS staging of R rows x DP columns.  A thread owns 16-byte chunks
// (8 columns of one row); consecutive lanes take consecutive chunks of a row, so a 128-bit
// LDS write cycle of eight lanes covers eight different chunk positions.  Fetching into
// registers and committing to LDS are separate so that the next tile's loads can be in
// flight while the current tile is used.
template <typename T, int R, int DP>
struct TileStager {
  static constexpr int CH = DP / 8;                     // chunks per row
  static constexpr int TASKS = R * CH;
  static constexpr int PER = TASKS / kAttnThreads;      // chunks per thread
  static constexpr int ROW_STEP = kAttnThreads / CH;    // rows between a thread's consecutive chunks
  static_assert(TASKS % kAttnThreads == 0 && kAttnThreads % CH == 0, "whole chunks per thread, one column per thread");
  uint4 v[PER];
  const T* src_;
  int64_t ld_;
  int next_;
  static __device__ __forceinline__ int row_of(int i) { return threadIdx.x / CH + i * ROW_STEP; }
  static __device__ __forceinline__ int chunk() { return threadIdx.x % CH; }

  // Starts a walk at row r0 of the matrix whose row r begins at base + r * ld (elements).
  __device__ __forceinline__ void begin(const T* __restrict__ base, int64_t ld, int r0) {
    ld_ = ld;
    next_ = r0;
    src_ = base + (r0 + row_of(0)) * ld + chunk() * 8;
#pragma unroll
    for (int i = 0; i < PER; ++i) v[i] = make_uint4(0, 0, 0, 0);
  }
  // Fetches the next tile of the walk: rows >= r_end and columns >= D read as zero.  A tile
  // that lies inside the matrix takes the short path, unconditional loads from a pointer that
  // advances by a constant (chunks of padding columns never load and keep their zeros); only
  // the ragged last tile pays for per-row bounds checks.
  __device__ __forceinline__ void fetch_next(int r_end, int D) {
    if (chunk() * 8 < D) {
      if (next_ + R <= r_end) {
#pragma unroll
        for (int i = 0; i < PER; ++i) v[i] = *reinterpret_cast<const uint4*>(src_ + i * ROW_STEP * ld_);
      } else {
#pragma unroll
        for (int i = 0; i < PER; ++i)
          v[i] = next_ + row_of(i) < r_end ? *reinterpret_cast<const uint4*>(src_ + i * ROW_STEP * ld_)
                                           : make_uint4(0, 0, 0, 0);
      }
    }
    src_ += R * ld_;
    next_ += R;
  }
  __device__ __forceinline__ void commit(char* __restrict__ lds) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) *reinterpret_cast<uint4*>(lds + tile_chunk_at<DP>(row_of(i), chunk())) = v[i];
  }
};

// Where a lane reads its fragments inside a staged tile, as byte offsets that depend on the
// lane only; everything else (which 32-row block, which 16 rows, which tile copy) is a
// compile-time or wave-uniform addend, so the fragment reads of a whole step share these few
// address registers.  That works because a row's swizzle depends only on r % 8, and the rows
// a lane reads differ from its first one by multiples of 8.
template <int DP>
struct TileLane {
  int rows[DP / 16];  // per 16-column slice ks: row lane%32, columns ks*16 + (lane/32)*8 .. +7
  int tr[DP / 32];    // per 32-column block dt: row 4*(lane/32) + (lane%16)/4, columns dt*32 + ((lane/16)%2)*16 + 4*(lane%4) .. +3
  __device__ __forceinline__ explicit TileLane(int lane) {
#pragma unroll
    for (int ks = 0; ks < DP / 16; ++ks) rows[ks] = tile_chunk_at<DP>(lane % 32, ks * 2 + lane / 32);
    const int col = ((lane / 16) % 2) * 16 + 4 * (lane % 4);
#pragma unroll
    for (int dt = 0; dt < DP / 32; ++dt)
      tr[dt] = tile_chunk_at<DP>(4 * (lane / 32) + (lane % 16) / 4, (dt * 32 + col) / 8) + (col % 8) * 2;
  }
};

// A operand for a product that contracts over the tile's columns: rows rt*32 + lane%32,
// columns ks*16 + (lane/32)*8 .. +7.
template <int DP>
__device__ __forceinline__ uint4 frag_rows(const char* __restrict__ lds, const TileLane<DP>& at, int rt, int ks) {
  return *reinterpret_cast<const uint4*>(lds + at.rows[ks] + rt * 32 * tile_row_bytes<DP>());
}

// A operand for a product that contracts over the tile's rows: MFMA row = tile column
// dt*32 + lane%32; k-slot e of lane half h stands for tile row t*16 + (e/4)*8 + 4h + e%4, the
// same assignment the score tile's registers have (see frag_from_acc).  Read with
// ds_read_b64_tr_b16: within 16 lanes, lane i supplies the address of four consecutive
// columns 4*(i%4).. of row i/4 of a 4 x 16 block and receives the four rows of column i.
template <int DP>
__device__ __forceinline__ uint4 frag_transposed(const char* __restrict__ lds, const TileLane<DP>& at, int dt, int t) {
  using lds_i16x4 = __attribute__((address_space(3))) short4_t;
  const char* p = lds + at.tr[dt] + t * 16 * tile_row_bytes<DP>();
  const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_i16x4*>(reinterpret_cast<uintptr_t>(p)));
  const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      reinterpret_cast<lds_i16x4*>(reinterpret_cast<uintptr_t>(p + 8 * tile_row_bytes<DP>())));
  const uint2 l = __builtin_bit_cast(uint2, lo), h = __builtin_bit_cast(uint2, hi);
  return make_uint4(l.x, l.y, h.x, h.y);
}

// B operand from a 32x32 accumulator tile: registers 8*half .. 8*half+7, i.e. rows
// half*16 + (e/4)*8 + 4*(lane/32) + e%4 of column lane%32.
template <typename T>
__device__ __forceinline__ uint4 frag_from_acc(const floatx16& acc, int half) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = Mma<T>::pack2(acc[half * 8 + 2 * i], acc[half * 8 + 2 * i + 1]);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// Row index inside a 32-row tile of accumulator register r.
__device__ __forceinline__ int acc_row(int r, int lane) { return (r / 4) * 8 + (lane / 32) * 4 + (r % 4); }

__device__ __forceinline__ floatx16 zero16() {
  floatx16 z;
#pragma unroll
  for (int r = 0; r < 16; ++r) z[r] = 0.f;
  return z;
}

// The two lanes that share a query (lane and lane ^ 32) exchange a value with one
// v_permlane32_swap instead of a round trip through LDS (ds_bpermute): afterwards `lo` holds
// lanes 0..31 of v in both halves of the wave and `hi` lanes 32..63.  The no-ops cover the
// wait states between a VALU write of the operands, the swap, and a VALU read of the
// results, which the compiler cannot see inside the asm.
__device__ __forceinline__ void split_halves(float v, float& lo, float& hi) {
  lo = v;
  hi = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
}
__device__ __forceinline__ float max_halves(float v) {
  float lo, hi;
  split_halves(v, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float sum_halves(float v) {
  float lo, hi;
  split_halves(v, lo, hi);
  return lo + hi;
}

// Packed store of four consecutive accumulator registers (four consecutive d) times `f`.
template <typename T>
__device__ __forceinline__ void store4(T* dst, const floatx16& acc, int g, float f) {
  uint2 w;
  w.x = Mma<T>::pack2(acc[g * 4] * f, acc[g * 4 + 1] * f);
  w.y = Mma<T>::pack2(acc[g * 4 + 2] * f, acc[g * 4 + 3] * f);
  *reinterpret_cast<uint2*>(dst) = w;
}

// Additive bias (B, H, S, S): in the forward and the dQ walk a lane keeps one query row and its
// accumulator registers run over keys in groups of four consecutive ones, so the bias of a
// group is one 8-byte load where the row allows it (S a multiple of 4, the tensor 8-byte
// aligned, the group inside the row); the two lanes of a row then read whole 16-byte pieces
// and, over a step's eight groups, exactly the row's 128 bytes.  (Element by element, 32
// two-byte loads per lane and step, the forward ran at 0.7 TB/s of bias: 1.10 ms at B2 H12
// S4096 against 0.17 ms without a bias.)
template <typename T>
__device__ __forceinline__ float bias_at(const uint2& w, int j) {
  T h[4];
  __builtin_memcpy(h, &w, 8);
  return to_float(h[j]);
}
__device__ __forceinline__ bool bias_rows_vectorise(const void* mask, int S) {
  return S % 4 == 0 && reinterpret_cast<uintptr_t>(mask) % 8 == 0;
}
// row[n .. n + 3] as four packed 16-bit values; `packed`: one 8-byte load, else element by element
// with the index clamped to the row (the values past its end are never used).
template <typename T>
__device__ __forceinline__ uint2 bias_group(const T* __restrict__ row, int n, int S, bool packed) {
  static_assert(sizeof(T) == 2, "16-bit tensors");
  if (packed) return *reinterpret_cast<const uint2*>(row + n);
  const uint16_t* raw = reinterpret_cast<const uint16_t*>(row);
  uint2 w;
  w.x = raw[min(n, S - 1)] | static_cast<uint32_t>(raw[min(n + 1, S - 1)]) << 16;
  w.y = raw[min(n + 2, S - 1)] | static_cast<uint32_t>(raw[min(n + 3, S - 1)]) << 16;
  return w;
}

// ---- forward -----------------------------------------------------------------------------

template <typename T, int DP, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(kAttnThreads, DP <= 128 ? 2 : 1) void attn_fwd_mfma_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                                        const T* __restrict__ v,
                                                                        const T* __restrict__ mask, T* __restrict__ o,
                                                                        float* __restrict__ lse, AttnDims a, float scale) {
  constexpr int BM = 128, BN = 64, KS = DP / 16, DT = DP / 32;
  // Two copies of each staged tile: step i computes from copy i % 2 while the tile of step
  // i + 1 is written into the other, so one barrier per step suffices.
  __shared__ __attribute__((aligned(16))) char k_rows_s[2][BN * tile_row_bytes<DP>()];
  __shared__ __attribute__((aligned(16))) char v_rows_s[2][BN * tile_row_bytes<DP>()];

  const int nqb = (a.S + BM - 1) / BM;
  // Consecutive workgroups go to different XCDs, so the (batch, head) index varies fastest:
  // every XCD then gets the same mix of query blocks, and the blocks of one (batch, head)
  // share one XCD's L2 when B*H is a multiple of the XCD count.  Causal: later query
  // blocks visit more keys; all of them launch first.
  const int n_bh = a.B * a.H;
  const int qb = CAUSAL ? nqb - 1 - blockIdx.x / n_bh : blockIdx.x / n_bh;
  const int h = (blockIdx.x % n_bh) % a.H;
  const int b = (blockIdx.x % n_bh) / a.H;
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int half = lane / 32;
  const TileLane<DP> at(lane);
  const int m_wave = qb * BM + wave * 32;
  const int m = m_wave + lane % 32;
  const int64_t ld = a.ld;  // token stride of Q, K, V
  const T* kbase = k + qkv_at(a, b, 0, h);
  const T* vbase = v + qkv_at(a, b, 0, h);

  uint4 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 16 + half * 8;
    qf[ks] = (m < a.S && d < a.D) ? *reinterpret_cast<const uint4*>(q + qkv_at(a, b, m, h) + d) : make_uint4(0, 0, 0, 0);
    settle(qf[ks]);
  }
  floatx16 acc_o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) acc_o[dt] = zero16();
  float m_run = -INFINITY, l_run = 0.f;
  const float c = scale * kAttnLog2e;
  const T* mrow = HAS_BIAS ? mask + ((static_cast<int64_t>(b) * a.H + h) * a.S + min(m, a.S - 1)) * a.S : nullptr;
  const bool bias_vec = HAS_BIAS && bias_rows_vectorise(mask, a.S);

  const int n_end = CAUSAL ? min(a.S, qb * BM + BM) : a.S;
  TileStager<T, BN, DP> ks_stage, vs_stage;
  ks_stage.begin(kbase, ld, 0);
  vs_stage.begin(vbase, ld, 0);
  ks_stage.fetch_next(a.S, a.D);
  vs_stage.fetch_next(a.S, a.D);
  ks_stage.commit(k_rows_s[0]);
  vs_stage.commit(v_rows_s[0]);
  if (BN < n_end) {
    ks_stage.fetch_next(a.S, a.D);
    vs_stage.fetch_next(a.S, a.D);
  }
  int cur = 0;
  for (int n0 = 0; n0 < n_end; n0 += BN, cur ^= 1) {
    // Copy `cur` is complete and every wave has finished reading the other copy.
    __syncthreads();
    if (n0 + BN < n_end) {
      ks_stage.commit(k_rows_s[cur ^ 1]);
      vs_stage.commit(v_rows_s[cur ^ 1]);
      if (n0 + 2 * BN < n_end) {
        ks_stage.fetch_next(a.S, a.D);
        vs_stage.fetch_next(a.S, a.D);
      }
    }
    const char* k_rows = k_rows_s[cur];
    const char* v_rows = v_rows_s[cur];
    if (CAUSAL && n0 > m_wave + 31) continue;  // every key of the block is in this wave's future

    // The step's bias: requested before the score products where the registers allow (narrow
    // heads), else tile by tile where it is used.
    constexpr bool BIAS_EARLY = DP <= 64;
    uint2 bias_w[2][4];
    const bool bias_packed = bias_vec && n0 + BN <= a.S;
    auto load_bias = [&](int nt) {
#pragma unroll
      for (int g = 0; g < 4; ++g) bias_w[nt][g] = bias_group<T>(mrow, n0 + nt * 32 + g * 8 + half * 4, a.S, bias_packed);
    };
    if (HAS_BIAS && BIAS_EARLY) {
      load_bias(0);
      load_bias(1);
    }

    floatx16 s[2];
    // The forward is bound by its VALU work (32 exponentials and about 150 other VALU
    // instructions per 16 MFMAs and wave), three waves per SIMD: a wave that is issuing MFMAs
    // gets priority over the ones doing softmax arithmetic, which keeps the matrix pipe fed
    // (3-4 % faster; the same hints in the backward kernels measured neutral to slower).
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      s[nt] = zero16();
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) s[nt] = Mma<T>::run(frag_rows<DP>(k_rows, at, nt, ks), qf[ks], s[nt]);
    }
    __builtin_amdgcn_s_setprio(0);
    // A block needs per-element masking only at the end of the sequence and, for causal
    // attention, where it crosses the diagonal of this wave's queries.
    const bool plain = !HAS_BIAS && c > 0.f && n0 + BN <= a.S && (!CAUSAL || n0 + BN - 1 <= m_wave);
    float corr;
    if (plain) {
      float mx = s[0][0];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[nt][r]);
      mx = max_halves(mx) * c;
      const float m_new = fmaxf(m_run, mx);
      corr = fexp2(m_run - m_new);
      float lsum = 0.f;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fexp2(fmaf(s[nt][r], c, -m_new));
          s[nt][r] = p;
          lsum += p;
        }
      lsum = sum_halves(lsum);
      l_run = l_run * corr + lsum;
      m_run = m_new;
    } else {
      float mx = -INFINITY;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        if (HAS_BIAS && !BIAS_EARLY) load_bias(nt);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int n = n0 + nt * 32 + acc_row(r, lane);
          bool valid = n < a.S;
          if (CAUSAL) valid = valid && n <= m;
          float sv = s[nt][r] * c;
          if (HAS_BIAS) sv = fmaf(bias_at<T>(bias_w[nt][r / 4], r % 4), kAttnLog2e, sv);
          sv = valid ? sv : -INFINITY;
          s[nt][r] = sv;
          mx = fmaxf(mx, sv);
        }
      }
      mx = max_halves(mx);
      const float m_new = fmaxf(m_run, mx);
      // m_new is -inf only for rows past the end of the sequence (all their keys masked)
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      corr = fexp2(m_run - m_use);
      float lsum = 0.f;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fexp2(s[nt][r] - m_use);
          s[nt][r] = p;
          lsum += p;
        }
      lsum = sum_halves(lsum);
      l_run = l_run * corr + lsum;
      m_run = m_new;
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc_o[dt][r] *= corr;
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int t = 0; t < BN / 16; ++t) {
      const uint4 pf = frag_from_acc<T>(s[t / 2], t % 2);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) acc_o[dt] = Mma<T>::run(frag_transposed<DP>(v_rows, at, dt, t), pf, acc_o[dt]);
    }
    __builtin_amdgcn_s_setprio(0);
  }

  if (m < a.S) {
    const float inv = 1.0f / l_run;
    T* orow = o + o_at(a, b, h, m);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = dt * 32 + g * 8 + half * 4;
        if (d < a.D) store4<T>(orow + d, acc_o[dt], g, inv);
      }
    if (half == 0) lse[(static_cast<int64_t>(b) * a.H + h) * a.S + m] = m_run * kAttnLn2 + logf(l_run);
  }
}

// ---- dQ ----------------------------------------------------------------------------------
// A wave owns MQ tiles of 32 queries; every A fragment read from LDS (K rows, V rows,
// K^T) feeds MQ MFMAs, which is what keeps LDS bandwidth below the MFMA rate.

// Head dims above 128 (the 256 bucket): the backward walks of a block run as this many
// workgroups, each producing one part of the head dimension of its gradients.
constexpr int kAttnWideSplit = 2;

// Bytes of LDS the dQ walk stages its tiles in.
template <int DP>
constexpr int dq_lds_bytes() {
  return (DP <= 64 ? 2 : 1) * 2 * 64 * tile_row_bytes<DP>();  // copies of a K tile and a V tile
}

// The work of workgroup `block` of a dQ launch; `smem` holds dq_lds_bytes<DP>() bytes.
// DSPLIT > 1: the workgroup produces only part DPART of the head dimension's DSPLIT equal
// parts of dQ (the score products still run over the whole head), so that the accumulators of a
// 256-wide head fit the register file; the parts are separate workgroups.
template <typename T, int DP, int MQ, bool CAUSAL, bool HAS_BIAS, int DSPLIT = 1, int DPART = 0>
__device__ __forceinline__ void attn_dq_block(const int block, char* smem, const T* __restrict__ d_o,
                                              const T* __restrict__ q, const T* __restrict__ k,
                                              const T* __restrict__ v, const T* __restrict__ mask,
                                              const float* __restrict__ lse, const float* __restrict__ delta,
                                              T* __restrict__ dq, const AttnDims& a, float scale) {
  constexpr int BM = 128 * MQ, BN = 64, KS = DP / 16, DT = DP / 32 / DSPLIT, DT0 = DPART * DT;
  static_assert((DP / 32) % DSPLIT == 0 && DPART < DSPLIT, "parts of the head dimension");
  // Two copies of each staged tile (step i computes from copy i % 2 while the tile of step
  // i + 1 is written into the other: one barrier per step) for head dims up to 64.  Above,
  // one copy and two barriers per step: the two-copy schedule spills more there (68-108 bytes
  // per lane against 44-80) and measured 20-30 % slower.
  constexpr int NBUF = DP <= 64 ? 2 : 1;
  constexpr int ROWS = BN * tile_row_bytes<DP>();
  auto k_rows_s = reinterpret_cast<char(*)[ROWS]>(smem);
  auto v_rows_s = reinterpret_cast<char(*)[ROWS]>(smem + NBUF * ROWS);
  static_assert(dq_lds_bytes<DP>() == 2 * NBUF * ROWS, "LDS size");

  const int nqb = (a.S + BM - 1) / BM;
  // (batch, head) varies fastest across consecutive workgroups, heaviest query blocks first.
  const int n_bh = a.B * a.H;
  const int qb = CAUSAL ? nqb - 1 - block / n_bh : block / n_bh;
  const int h = (block % n_bh) % a.H;
  const int b = (block % n_bh) / a.H;
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int half = lane / 32;
  const TileLane<DP> at(lane);
  const int m_wave = qb * BM + wave * (32 * MQ);
  const int64_t ld = a.ld;
  const T* kbase = k + qkv_at(a, b, 0, h);
  const T* vbase = v + qkv_at(a, b, 0, h);
  const int64_t bh = static_cast<int64_t>(b) * a.H + h;

  // Q is held pre-multiplied by scale * log2(e), and the score and dP products start from
  // accumulators holding -lse (log2 units) and -delta, this lane's query being the same
  // for every tile: the matrix core then delivers S*c - lse and dP - delta directly.
  const float c = scale * kAttnLog2e;
  int m[MQ];
  uint4 qf[MQ][KS], dof[MQ][KS];
  float lse2[MQ], dl[MQ];
  floatx16 s_init[MQ], dp_init[MQ];
  const T* mrow[MQ];
  floatx16 acc[MQ][DT];
#pragma unroll
  for (int mq = 0; mq < MQ; ++mq) {
    m[mq] = m_wave + mq * 32 + lane % 32;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 16 + half * 8;
      const bool ok = m[mq] < a.S && d < a.D;
      qf[mq][ks] = ok ? *reinterpret_cast<const uint4*>(q + qkv_at(a, b, m[mq], h) + d) : make_uint4(0, 0, 0, 0);
      qf[mq][ks] = scale_frag<T>(qf[mq][ks], c);
      dof[mq][ks] = ok ? *reinterpret_cast<const uint4*>(d_o + o_at(a, b, h, m[mq]) + d) : make_uint4(0, 0, 0, 0);
      settle(dof[mq][ks]);
    }
    // Rows past the end get lse = +inf so that their probabilities vanish.
    lse2[mq] = m[mq] < a.S ? lse[bh * a.S + m[mq]] * kAttnLog2e : INFINITY;
    dl[mq] = m[mq] < a.S ? delta[bh * a.S + m[mq]] : 0.f;
    mrow[mq] = HAS_BIAS ? mask + (bh * a.S + min(m[mq], a.S - 1)) * a.S : nullptr;
    s_init[mq] = splat16(-lse2[mq]);
    dp_init[mq] = splat16(-dl[mq]);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[mq][dt] = zero16();
  }

  const bool bias_vec = HAS_BIAS && bias_rows_vectorise(mask, a.S);
  const int n_end = CAUSAL ? min(a.S, qb * BM + BM) : a.S;
  TileStager<T, BN, DP> ks_stage, vs_stage;
  ks_stage.begin(kbase, ld, 0);
  vs_stage.begin(vbase, ld, 0);
  ks_stage.fetch_next(a.S, a.D);
  vs_stage.fetch_next(a.S, a.D);
  if constexpr (NBUF == 2) {
    ks_stage.commit(k_rows_s[0]);
    vs_stage.commit(v_rows_s[0]);
    if (BN < n_end) {
      ks_stage.fetch_next(a.S, a.D);
      vs_stage.fetch_next(a.S, a.D);
    }
  }
  // The bias of a step's two key tiles, as packed groups (bias_group).  Narrow heads have the
  // registers to request it a whole step ahead, like the K and V tiles; wide heads load it tile
  // by tile where it is used.
  constexpr bool BIAS_AHEAD = HAS_BIAS && DP <= 64;
  uint2 bias_cur[MQ][BN / 32][4], bias_nxt[MQ][BN / 32][4];
  auto load_bias_step = [&](int n0, uint2 (&dst)[MQ][BN / 32][4]) {
    const bool packed = bias_vec && n0 + BN <= a.S;
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
      for (int nt = 0; nt < BN / 32; ++nt)
#pragma unroll
        for (int g = 0; g < 4; ++g) dst[mq][nt][g] = bias_group<T>(mrow[mq], n0 + nt * 32 + g * 8 + half * 4, a.S, packed);
  };
  if constexpr (BIAS_AHEAD) load_bias_step(0, bias_nxt);
  int cur = 0;
  for (int n0 = 0; n0 < n_end; n0 += BN, cur ^= (NBUF - 1)) {
    if constexpr (BIAS_AHEAD) {
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
        for (int nt = 0; nt < BN / 32; ++nt)
#pragma unroll
          for (int g = 0; g < 4; ++g) bias_cur[mq][nt][g] = bias_nxt[mq][nt][g];
      if (n0 + BN < n_end) load_bias_step(n0 + BN, bias_nxt);
    }
    if constexpr (NBUF == 2) {
      // Copy `cur` is complete and every wave has finished reading the other copy.
      __syncthreads();
      if (n0 + BN < n_end) {
        ks_stage.commit(k_rows_s[cur ^ 1]);
        vs_stage.commit(v_rows_s[cur ^ 1]);
        if (n0 + 2 * BN < n_end) {
          ks_stage.fetch_next(a.S, a.D);
          vs_stage.fetch_next(a.S, a.D);
        }
      }
    } else {
      __syncthreads();  // every wave has finished reading the previous tile
      ks_stage.commit(k_rows_s[0]);
      vs_stage.commit(v_rows_s[0]);
      __syncthreads();
      if (n0 + BN < n_end) {
        ks_stage.fetch_next(a.S, a.D);
        vs_stage.fetch_next(a.S, a.D);
      }
    }
    const char* k_rows = k_rows_s[cur];
    const char* v_rows = v_rows_s[cur];
    if (CAUSAL && n0 > m_wave + 32 * MQ - 1) continue;  // every key of the block is in this wave's future

    // One 32-key tile at a time: S^T and dP^T for all MQ query tiles, dS^T in place, then
    // its contribution to dQ^T.
#pragma unroll
    for (int nt = 0; nt < BN / 32; ++nt) {
      floatx16 s[MQ], dp[MQ];
      uint2 bias_w[MQ][4];
      const bool bias_packed = bias_vec && n0 + nt * 32 + 32 <= a.S;
      auto load_bias = [&](int mq) {
#pragma unroll
        for (int g = 0; g < 4; ++g)
          bias_w[mq][g] = bias_group<T>(mrow[mq], n0 + nt * 32 + g * 8 + half * 4, a.S, bias_packed);
      };
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq) {
        s[mq] = s_init[mq];
        dp[mq] = dp_init[mq];
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const uint4 ka = frag_rows<DP>(k_rows, at, nt, ks);
        const uint4 va = frag_rows<DP>(v_rows, at, nt, ks);
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq) {
          s[mq] = Mma<T>::run(ka, qf[mq][ks], s[mq]);
          dp[mq] = Mma<T>::run(va, dof[mq][ks], dp[mq]);
        }
      }
      const int nb = n0 + nt * 32;
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq) {
        const bool plain = !HAS_BIAS && nb + 32 <= a.S && (!CAUSAL || nb + 31 <= m_wave + mq * 32);
        if (plain) {
#pragma unroll
          for (int r = 0; r < 16; ++r) s[mq][r] = fexp2(s[mq][r]) * dp[mq][r];
        } else {
          if (HAS_BIAS && !BIAS_AHEAD) load_bias(mq);
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int n = nb + acc_row(r, lane);
            bool valid = n < a.S;
            if (CAUSAL) valid = valid && n <= m[mq];
            float sv = s[mq][r];
            if (HAS_BIAS) {
              const uint2 w = BIAS_AHEAD ? bias_cur[mq][nt][r / 4] : bias_w[mq][r / 4];
              sv = fmaf(bias_at<T>(w, r % 4), kAttnLog2e, sv);
            }
            float p = fexp2(sv);
            p = valid ? p : 0.f;
            s[mq][r] = p * dp[mq][r];  // dS^T
          }
        }
      }
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const int t = nt * 2 + hf;
        uint4 dsf[MQ];
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq) dsf[mq] = frag_from_acc<T>(s[mq], hf);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const uint4 kt = frag_transposed<DP>(k_rows, at, DT0 + dt, t);
#pragma unroll
          for (int mq = 0; mq < MQ; ++mq) acc[mq][dt] = Mma<T>::run(kt, dsf[mq], acc[mq][dt]);
        }
      }
    }
  }

#pragma unroll
  for (int mq = 0; mq < MQ; ++mq) {
    if (m[mq] < a.S) {
      T* out = dq + qkv_at(a, b, m[mq], h);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int d = (DT0 + dt) * 32 + g * 8 + half * 4;
          if (d < a.D) store4<T>(out + d, acc[mq][dt], g, scale);
        }
    }
  }
}

// ---- dK, dV ------------------------------------------------------------------------------

// Bytes of LDS the dK/dV walk stages its tiles and row statistics in.
// Bytes of LDS the dK/dV walk stages its tiles and row statistics in, for steps of BQ queries:
// two copies of a Q tile, a dO tile, lse and delta.
template <int DP, int BQ>
constexpr int dkdv_lds_bytes() {
  return 2 * (2 * BQ * tile_row_bytes<DP>() + 2 * BQ * 4);
}
// Queries per step when the walk has a launch of its own (sequences past 1024 tokens, or head
// dims above 64): 128 for head dims up to 64, half as many barriers per query (S = 4096
// 440 -> 430 us, S = 2048 causal 198 -> 191 us; at S = 256 it would cost 3 %, but there the
// walk shares a launch with dQ and steps by 64).
template <int DP>
constexpr int dkdv_long_step() { return DP <= 64 ? 128 : 64; }

// The work of workgroup `block` of a dK/dV launch, BQ queries per step; `smem` holds
// dkdv_lds_bytes<DP, BQ>() bytes.
// DSPLIT, DPART: as for attn_dq_block, for dK and dV.
template <typename T, int DP, int BQ, bool CAUSAL, bool HAS_BIAS, int DSPLIT = 1, int DPART = 0>
__device__ __forceinline__ void attn_dkdv_block(const int block, char* smem, const T* __restrict__ d_o,
                                                const T* __restrict__ q, const T* __restrict__ k,
                                                const T* __restrict__ v, const T* __restrict__ mask,
                                                const float* __restrict__ lse, const float* __restrict__ delta,
                                                T* __restrict__ dk, T* __restrict__ dv, const AttnDims& a,
                                                float scale) {
  constexpr int BNK = 128;                 // keys per workgroup
  constexpr int MT = BQ / 32, KS = DP / 16, DT = DP / 32 / DSPLIT, DT0 = DPART * DT;
  static_assert((DP / 32) % DSPLIT == 0 && DPART < DSPLIT, "parts of the head dimension");
  // Two copies of every staged tile: step i computes from copy i % 2 while the tile of step
  // i + 1 is written into the other, so one barrier per step suffices.
  constexpr int ROWS = BQ * tile_row_bytes<DP>();
  auto q_rows_s = reinterpret_cast<char(*)[ROWS]>(smem);
  auto do_rows_s = reinterpret_cast<char(*)[ROWS]>(smem + 2 * ROWS);
  auto lse_ss = reinterpret_cast<float(*)[BQ]>(smem + 4 * ROWS);
  auto delta_ss = reinterpret_cast<float(*)[BQ]>(smem + 4 * ROWS + 2 * BQ * 4);
  static_assert(dkdv_lds_bytes<DP, BQ>() == 4 * ROWS + 4 * BQ * 4, "LDS size");

  // (batch, head) varies fastest across consecutive workgroups.  Causal: earlier key blocks
  // are seen by more queries; all of them launch first.
  const int n_bh = a.B * a.H;
  const int kb = block / n_bh;
  const int h = (block % n_bh) % a.H;
  const int b = (block % n_bh) / a.H;
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int half = lane / 32;
  const TileLane<DP> at(lane);
  const int n_wave = kb * BNK + wave * 32;
  const int n = n_wave + lane % 32;
  const int64_t ld = a.ld;
  const T* qbase = q + qkv_at(a, b, 0, h);
  const T* dobase = d_o + o_at(a, b, h, 0);
  const int64_t bh = static_cast<int64_t>(b) * a.H + h;

  uint4 kf[KS], vf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 16 + half * 8;
    const bool ok = n < a.S && d < a.D;
    kf[ks] = ok ? *reinterpret_cast<const uint4*>(k + qkv_at(a, b, n, h) + d) : make_uint4(0, 0, 0, 0);
    // K is held pre-multiplied by scale * log2(e): the score product then comes out in the
    // exponent's units.  (dK is formed from the unscaled Q tile, so nothing else changes.)
    kf[ks] = scale_frag<T>(kf[ks], scale * kAttnLog2e);
    vf[ks] = ok ? *reinterpret_cast<const uint4*>(v + qkv_at(a, b, n, h) + d) : make_uint4(0, 0, 0, 0);
    settle(vf[ks]);
  }
  floatx16 acc_k[DT], acc_v[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    acc_k[dt] = zero16();
    acc_v[dt] = zero16();
  }

  // Causal: queries before the workgroup's first key see none of its keys.
  const int m_begin = CAUSAL ? (kb * BNK / BQ) * BQ : 0;
  TileStager<T, BQ, DP> q_stage, do_stage;
  float lse_next, delta_next;
  q_stage.begin(qbase, ld, m_begin);
  do_stage.begin(dobase, o_ld(a), m_begin);
  // Global -> registers for the next step of the walk, which starts at query m.
  // The row statistics go first: the compiler guards the reuse of their registers with a
  // wait for every load issued before it, which must not include this step's tile loads.
  auto fetch_step = [&](int m) {
    lse_next = INFINITY;
    delta_next = 0.f;
    if (threadIdx.x < BQ && m + threadIdx.x < a.S) {
      lse_next = lse[bh * a.S + m + threadIdx.x];  // scaled to log2 units when it is committed
      delta_next = delta[bh * a.S + m + threadIdx.x];
    }
    q_stage.fetch_next(a.S, a.D);
    do_stage.fetch_next(a.S, a.D);
  };
  // Registers -> LDS copy `buf`.
  auto commit_step = [&](int buf) {
    q_stage.commit(q_rows_s[buf]);
    do_stage.commit(do_rows_s[buf]);
    if (threadIdx.x < BQ) {
      // Stored negated: they initialise the accumulators of the S and dP products.  Rows
      // past the end carry -lse = -inf (their probabilities vanish) and delta = 0.
      lse_ss[buf][threadIdx.x] = -lse_next * kAttnLog2e;
      delta_ss[buf][threadIdx.x] = -delta_next;
    }
  };
  fetch_step(m_begin);
  commit_step(0);
  if (m_begin + BQ < a.S) fetch_step(m_begin + BQ);
  int cur = 0;
  for (int m0 = m_begin; m0 < a.S; m0 += BQ, cur ^= 1) {
    // Copy `cur` is complete and every wave has finished reading the other copy.
    __syncthreads();
    if (m0 + BQ < a.S) {
      commit_step(cur ^ 1);
      if (m0 + 2 * BQ < a.S) fetch_step(m0 + 2 * BQ);
    }
    const char* q_rows = q_rows_s[cur];
    const char* do_rows = do_rows_s[cur];
    const float* lse_s = lse_ss[cur];
    const float* delta_s = delta_ss[cur];
    if (CAUSAL && m0 + BQ - 1 < n_wave) continue;  // all of this step's queries precede the wave's keys

    // Per-element masking is needed only for key columns past the end and where the step
    // crosses the diagonal of this wave's keys.
    const bool plain = !HAS_BIAS && n_wave + 31 < a.S && (!CAUSAL || n_wave + 31 <= m0);
    // One 32-query tile at a time: S and dP (column = this lane's key, rows = queries),
    // then P and dS in place, then their contributions to dV and dK.  LDS fragments are
    // fetched a phase ahead (the transposed ones, and the next tile's row fragments, while
    // the exponentials run) so that no MFMA waits on an LDS read it has just issued.
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      // Accumulators start at -lse and -delta of their rows (register r <-> query row
      // (r/4)*8 + half*4 + r%4): the products deliver S*c - lse and dP - delta.
      floatx16 s, dp;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float4 l4 = *reinterpret_cast<const float4*>(&lse_s[mt * 32 + g * 8 + half * 4]);
        const float4 d4 = *reinterpret_cast<const float4*>(&delta_s[mt * 32 + g * 8 + half * 4]);
        s[g * 4 + 0] = l4.x; s[g * 4 + 1] = l4.y; s[g * 4 + 2] = l4.z; s[g * 4 + 3] = l4.w;
        dp[g * 4 + 0] = d4.x; dp[g * 4 + 1] = d4.y; dp[g * 4 + 2] = d4.z; dp[g * 4 + 3] = d4.w;
      }
      // The tile's bias: this lane's key column of sixteen query rows, two bytes each (a half
      // wave reads 64 contiguous bytes of a row), requested before the products.  Clamped
      // addresses: always in bounds, the value is discarded where the element is invalid.
      T bias_v[16];
      if (HAS_BIAS) {
        const T* bcol = mask + bh * a.S * a.S + min(n, a.S - 1);
#pragma unroll
        for (int r = 0; r < 16; ++r)
          bias_v[r] = bcol[static_cast<int64_t>(min(m0 + mt * 32 + acc_row(r, lane), a.S - 1)) * a.S];
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        s = Mma<T>::run(frag_rows<DP>(q_rows, at, mt, ks), kf[ks], s);
        dp = Mma<T>::run(frag_rows<DP>(do_rows, at, mt, ks), vf[ks], dp);
      }
      // The transposed fragments of the second phase are fetched now, so that their LDS
      // latency runs under the exponentials instead of in front of each MFMA.
      uint4 tq[2][DT], tdo[2][DT];
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          tdo[hf][dt] = frag_transposed<DP>(do_rows, at, DT0 + dt, mt * 2 + hf);
          tq[hf][dt] = frag_transposed<DP>(q_rows, at, DT0 + dt, mt * 2 + hf);
        }
      __builtin_amdgcn_sched_barrier(0);
      if (plain) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fexp2(s[r]);
          s[r] = p;
          dp[r] = p * dp[r];
        }
      } else {
        // Same arithmetic on every element, then a select: no per-element branches.
        const bool col_ok = n < a.S;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int mm = m0 + mt * 32 + acc_row(r, lane);
          bool valid = col_ok;
          if (CAUSAL) valid = valid && n <= mm;
          float sv = s[r];
          if (HAS_BIAS) sv = fmaf(to_float(bias_v[r]), kAttnLog2e, sv);
          float p = fexp2(sv);  // rows past the end started from -inf: p = 0
          p = valid ? p : 0.f;
          s[r] = p;
          dp[r] = p * dp[r];
        }
      }
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const uint4 pf = frag_from_acc<T>(s, hf);
        const uint4 dsf = frag_from_acc<T>(dp, hf);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          acc_v[dt] = Mma<T>::run(tdo[hf][dt], pf, acc_v[dt]);
          acc_k[dt] = Mma<T>::run(tq[hf][dt], dsf, acc_k[dt]);
        }
      }
    }
  }

  if (n < a.S) {
    T* outk = dk + qkv_at(a, b, n, h);
    T* outv = dv + qkv_at(a, b, n, h);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = (DT0 + dt) * 32 + g * 8 + half * 4;
        if (d < a.D) {
          store4<T>(outk + d, acc_k[dt], g, scale);
          store4<T>(outv + d, acc_v[dt], g, 1.0f);
        }
      }
  }
}

// ---- dK, dV: software-pipelined walk (head dim <= 64, no bias) ----------------------------
// Same products and register layouts as attn_dkdv_block, scheduled so that a wave keeps the
// matrix pipe fed by itself.  The 32-query tiles of a walk form one sequence g = 0, 1, ...;
// per tile there are five stages:
//   L1(g)  LDS -> registers: the eight row fragments of Q and dO, and -lse / -delta of the
//          tile's rows straight into the S and dP accumulators
//   A(g)   eight MFMAs: S = Q K^T - lse, dP = dO V^T - delta
//   B(g)   VALU: P = exp2(S), dS = P (dP - delta), both rounded and packed
//   L2(g)  LDS -> registers: the transposed fragments of dO and Q
//   C(g)   eight MFMAs: dV^T += dO^T P, dK^T += Q^T dS
// and iteration g issues  [A(g+1) interleaved with B(g) and L2(g)]  then  [C(g) interleaved
// with L1(g+2)]: every MFMA's operands were requested a block earlier, and the exponentials
// of one tile run under the score products of the next.  S and dP alternate between two
// register sets.  The order is pinned with sched_barrier between MFMA-sized groups.
//
// Tiles are copied global memory -> LDS by global_load_lds (no staging registers), 64 queries
// per step into a ring of three buffers: the copies of step i + 2 are issued right after the
// barrier that publishes step i + 1, which every wave passes between the two blocks of its
// first tile of step i.  At that point nobody reads the buffer of step i - 1 any more, and the
// copies of step i + 1 have had a whole step to land, so one barrier per step suffices and
// nothing waits on it.  lse and delta arrive pre-negated (lse also in log2 units) and padded
// per (batch, head) to a multiple of 64 rows with -inf / 0, so that rows past the end of the
// sequence give P = 0 without any per-element test; their Q / dO rows are copies of the last
// row.  Causal: wave w's keys meet the diagonal in tile w of the walk (which starts at the
// workgroup's first key); it starts there, with the masked elements' S accumulators
// initialised to -inf, and every later tile is unmasked.

// f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N - 1>{}): a loop whose index is a
// compile-time constant inside the body (DPP controls are instruction immediates).
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}
// The value that lane J of this lane's own row of 16 lanes holds (DPP row_newbcast).
template <int J>
__device__ __forceinline__ float row_bcast(float v) {
  return dpp_move<0x150 + J>(v);
}

// The LDS image of the pipelined walks: as above, but chunk c of row r sits at position
// c ^ swz16(r) with swz16(r) = 4 * (r/2 % 2) + (r/4 % 2) + 2 * (r/8 % 2).  The 128-bit row reads
// of sixteen consecutive rows then fall on sixteen different bank groups (the plain swizzle
// serves them two rows per group, which doubles the cycles of half of all fragment reads),
// and the transposing reads stay conflict-free.  The price is that rows r and r + 8 no longer
// swizzle alike, so the second transposing read of a fragment has an address register of its
// own.  The tiles are written by global_load_lds, a kilobyte (eight rows) per wave
// instruction, so the image costs nothing on the way in.
__device__ __forceinline__ int tile_swz16(int r) { return 4 * ((r / 2) % 2) + (r / 4) % 2 + 2 * ((r / 8) % 2); }
template <int DP>
__device__ __forceinline__ int tile16_chunk_at(int r, int c) { return r * tile_row_bytes<DP>() + ((c ^ tile_swz16(r)) * 16); }
template <int DP>
struct TileLane16 {
  int rows[DP / 16];
  int tr_lo[DP / 32], tr_hi[DP / 32];
  __device__ __forceinline__ explicit TileLane16(int lane) {
#pragma unroll
    for (int ks = 0; ks < DP / 16; ++ks) rows[ks] = tile16_chunk_at<DP>(lane % 32, ks * 2 + lane / 32);
    const int col = ((lane / 16) % 2) * 16 + 4 * (lane % 4);
    const int r = 4 * (lane / 32) + (lane % 16) / 4;
#pragma unroll
    for (int dt = 0; dt < DP / 32; ++dt) {
      tr_lo[dt] = tile16_chunk_at<DP>(r, (dt * 32 + col) / 8) + (col % 8) * 2;
      tr_hi[dt] = tile16_chunk_at<DP>(r + 8, (dt * 32 + col) / 8) + (col % 8) * 2;
    }
  }
};
template <int DP>
__device__ __forceinline__ uint4 frag_rows(const char* __restrict__ lds, const TileLane16<DP>& at, int rt, int ks) {
  return *reinterpret_cast<const uint4*>(lds + at.rows[ks] + rt * 32 * tile_row_bytes<DP>());
}
template <int DP>
__device__ __forceinline__ uint4 frag_transposed(const char* __restrict__ lds, const TileLane16<DP>& at, int dt, int t) {
  using lds_i16x4 = __attribute__((address_space(3))) short4_t;
  const char* base = lds + t * 16 * tile_row_bytes<DP>();
  const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      reinterpret_cast<lds_i16x4*>(reinterpret_cast<uintptr_t>(base + at.tr_lo[dt])));
  const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      reinterpret_cast<lds_i16x4*>(reinterpret_cast<uintptr_t>(base + at.tr_hi[dt])));
  const uint2 l = __builtin_bit_cast(uint2, lo), h = __builtin_bit_cast(uint2, hi);
  return make_uint4(l.x, l.y, h.x, h.y);
}

template <int DP>
constexpr int dkdv_pipe_buf_bytes() {
  return 2 * 64 * tile_row_bytes<DP>() + 2 * 64 * 4;  // a Q tile, a dO tile, -lse, -delta of 64 queries
}
// Buffers in the ring of the pipelined walks: the copies of a step are issued kAttnRing - 1
// steps before the step is read.
#ifndef MG_ATTN_RING
#define MG_ATTN_RING 3
#endif
constexpr int kAttnRing = MG_ATTN_RING;
template <int DP>
constexpr int dkdv_pipe_lds_bytes() {
  return kAttnRing * dkdv_pipe_buf_bytes<DP>();
}

// s_waitcnt with only the vector-memory counter set (vmcnt in bits 3:0 and 15:14, the
// other counters left at "no wait").
#define MG_ATTN_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | 0x0f70)

__device__ __forceinline__ unsigned lds_address(const void* p) {
  using lds_ptr = __attribute__((address_space(3))) const char*;
  return static_cast<unsigned>(reinterpret_cast<uintptr_t>((lds_ptr)p));
}
// One wave-wide copy global -> LDS: lane l's 16 (or 4) bytes land at `lds_wave_base` + 16 l
// (4 l).  Written as assembly so that the compiler does not attach waits for these copies to
// unrelated LDS reads; m0 is used by nothing else in these kernels.
__device__ __forceinline__ void copy16_to_lds(unsigned lds_wave_base, const void* src) {
  const unsigned dst = __builtin_amdgcn_readfirstlane(lds_wave_base);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(src) : "memory");
}
__device__ __forceinline__ void copy4_to_lds(unsigned lds_wave_base, const void* src) {
  const unsigned dst = __builtin_amdgcn_readfirstlane(lds_wave_base);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(dst), "v"(src) : "memory");
}

// (The row statistics were also tried as one 4-byte LDS read per lane and tile, handed to
// the accumulator registers' rows by DPP row broadcasts inside stage B: eight fewer 16-byte LDS
// reads per tile, two more VALU operations per element, 226 us against 209 us for the S = 4096
// walk: the VALU is the scarcer resource here.)
constexpr bool kAttnStatDpp = false;
template <typename T, int DP, bool CAUSAL, bool STAT_DPP>
__device__ __forceinline__ void attn_dkdv_pipe_block(const int block, char* smem, const T* __restrict__ d_o,
                                                     const T* __restrict__ q, const T* __restrict__ k,
                                                     const T* __restrict__ v, const float* __restrict__ nlse,
                                                     const float* __restrict__ ndelta, const int s_pad,
                                                     T* __restrict__ dk, T* __restrict__ dv, const AttnDims& a,
                                                     float scale) {
  static_assert(DP == 64, "tile shapes below are written for a 64-wide head");
  constexpr int BNK = 128, BQ = 64, KS = DP / 16, DT = DP / 32;
  constexpr int ROWS = BQ * tile_row_bytes<DP>();
  constexpr int BUF = dkdv_pipe_buf_bytes<DP>();

  const int n_bh = a.B * a.H;
  const int kb = block / n_bh;
  const int h = (block % n_bh) % a.H;
  const int b = (block % n_bh) / a.H;
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int half = lane / 32;
  const TileLane16<DP> at(lane);
  const int n = kb * BNK + wave * 32 + lane % 32;
  const int64_t bh = static_cast<int64_t>(b) * a.H + h;

  uint4 kf[KS], vf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 16 + half * 8;
    const bool ok = n < a.S && d < a.D;
    kf[ks] = ok ? *reinterpret_cast<const uint4*>(k + qkv_at(a, b, n, h) + d) : make_uint4(0, 0, 0, 0);
    kf[ks] = scale_frag<T>(kf[ks], scale * kAttnLog2e);
    vf[ks] = ok ? *reinterpret_cast<const uint4*>(v + qkv_at(a, b, n, h) + d) : make_uint4(0, 0, 0, 0);
  }
  floatx16 acc_k[DT], acc_v[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    acc_k[dt] = zero16();
    acc_v[dt] = zero16();
  }

  const int m_begin = CAUSAL ? kb * BNK : 0;
  const int nsteps = (a.S - m_begin + BQ - 1) / BQ;
  const int G = 2 * nsteps;

  // ---- copies: step i -> buffer i % kAttnRing ----
  // Wave-instruction j of a tile covers its rows 8j .. 8j+7 (1 KB); this wave issues j = wave
  // and wave + 4 for Q and for dO.  Lane l writes chunk position l % 8 of row 8j + l / 8 and
  // therefore names the source chunk (l % 8) ^ swz16(row), with row % 16 = 8 (wave % 2) + l / 8.
  // A copy's address is a scalar base (the step's first row of this (batch, head)) plus a
  // 32-bit lane offset, so a step's copies cost two VALU operations each: the row, clamped to
  // the last row of the sequence, times the row pitch.  Chunks of padding columns (head
  // narrower than the tile) copy the row's chunk 0 instead: whatever lands in a padding column
  // of Q or dO only ever meets the zeros that K and V hold there.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int cp_row = lane / 8;
  const int cp_chunk = (lane % 8) ^ tile_swz16(8 * (wave % 2) + cp_row);  // rows 8j + cp_row, j = wave or wave + 4
  const unsigned cp_col_bytes = cp_chunk * 8 < a.D ? cp_chunk * 16 : 0;
  const char* q_bh = reinterpret_cast<const char*>(q + qkv_at(a, b, 0, h));
  const char* do_bh = reinterpret_cast<const char*>(d_o + o_at(a, b, h, 0));
  const unsigned q_pitch = static_cast<unsigned>(a.ld) * 2, do_pitch = static_cast<unsigned>(o_ld(a)) * 2;  // bytes per row
  const char* stat_bh = reinterpret_cast<const char*>((wave_u % 2 == 0 ? nlse : ndelta) + bh * s_pad);
  const unsigned smem_base = lds_address(smem);
  // Copy c of 5 of step `step` (clamped to the walk's last step: a copy past the end goes to a
  // buffer that nobody reads again) into buffer `buf`: Q rows, dO rows, Q rows, dO rows, a statistic.
  auto issue_piece = [&](int c, int step, int buf) {
    const int m0 = m_begin + min(step, nsteps - 1) * BQ;
    const unsigned base = smem_base + buf * BUF;
    if (c < 4) {
      const int jj = c / 2;
      const bool is_do = c % 2;
      const int j = wave_u + 4 * jj;
      const int row = min(8 * j + cp_row, a.S - 1 - m0);  // relative to m0
      const unsigned pitch = is_do ? do_pitch : q_pitch;
      const char* rows0 = (is_do ? do_bh : q_bh) + static_cast<int64_t>(m0) * pitch;
      const unsigned dst = __builtin_amdgcn_readfirstlane(base + (is_do ? ROWS : 0) + j * 1024);
      const unsigned off = row * pitch + cp_col_bytes;
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(rows0) : "memory");
    } else {
      const unsigned dst = __builtin_amdgcn_readfirstlane(base + 2 * ROWS + (wave_u % 2) * BQ * 4);
      const unsigned off = lane * 4;
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" ::"s"(dst), "v"(off), "s"(stat_bh + m0 * 4) : "memory");
    }
  };
  auto issue_step = [&](int step, int buf) {
#pragma unroll
    for (int c = 0; c < 5; ++c) issue_piece(c, step, buf);
  };

  // ---- stages ----
  floatx16 s[2], dp[2];
  float xs[2], xd[2];  // STAT_DPP: -lse and -delta of the tile's rows, spread over each row of 16 lanes
  uint4 qr[KS], dor[KS], tq[2][DT], tdo[2][DT], pf[2], dsf[2];
  uint32_t pw[8], dw[8];

  // LDS addresses of this lane's fragments, as running 32-bit values: `ra` (row fragments)
  // and `sa` (statistics) point into the buffer of the step that stage L1 reads, `tlo` / `thi`
  // (transposing reads) into the buffer of the step that stage L2 reads, and all of them
  // move on by one buffer at the end of every step.  Everything else about a read (Q or dO
  // tile, which 32 rows, which 16 rows) is an immediate offset of the instruction, so the
  // walk spends nine additions per step on addresses.
  typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
  using lds_u4 = __attribute__((address_space(3))) const uintx4*;
  typedef float floatx4 __attribute__((ext_vector_type(4)));
  using lds_f4 = __attribute__((address_space(3))) const floatx4*;
  using lds_f1 = __attribute__((address_space(3))) const float*;
  using lds_i16x4 = __attribute__((address_space(3))) short4_t*;
  unsigned ra[KS], sa, tlo[DT], thi[DT];
  // Accumulator register e of a 32 x 32 tile belongs to row (e/4)*8 + half*4 + e%4.
  // STAT_DPP: lane j of every row of 16 lanes fetches the statistics of exactly that row for
  // e = j, and stage B reads "its" value for register e from lane e of its own row of lanes
  // with a DPP broadcast (one 4-byte LDS read per lane and tile, two more VALU operations per
  // element).  Otherwise the S and dP accumulators start from -lse and -delta, read as eight
  // 16-byte broadcasts per tile.
  const int stat_row = ((lane % 16) / 4) * 8 + half * 4 + lane % 4;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) ra[ks] = smem_base + at.rows[ks];
  sa = smem_base + 2 * ROWS + (STAT_DPP ? stat_row * 4 : half * 16);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    tlo[dt] = smem_base + at.tr_lo[dt];
    thi[dt] = smem_base + at.tr_hi[dt];
  }
  int buf_l1 = 0, buf_l2 = 0;  // which buffer each group points into
  auto advance_l1 = [&]() {
    const int d = buf_l1 == kAttnRing - 1 ? -(kAttnRing - 1) * BUF : BUF;
    buf_l1 = buf_l1 == kAttnRing - 1 ? 0 : buf_l1 + 1;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ra[ks] += d;
    sa += d;
  };
  auto advance_l2 = [&]() {
    const int d = buf_l2 == kAttnRing - 1 ? -(kAttnRing - 1) * BUF : BUF;
    buf_l2 = buf_l2 == kAttnRing - 1 ? 0 : buf_l2 + 1;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      tlo[dt] += d;
      thi[dt] += d;
    }
  };
  auto read16 = [](unsigned addr) {
    const uintx4 x = *reinterpret_cast<lds_u4>(static_cast<uintptr_t>(addr));
    return make_uint4(x[0], x[1], x[2], x[3]);
  };
  auto read_tr = [](unsigned lo, unsigned hi) {
    const short4_t l4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_i16x4>(static_cast<uintptr_t>(lo)));
    const short4_t h4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_i16x4>(static_cast<uintptr_t>(hi)));
    const uint2 l = __builtin_bit_cast(uint2, l4), h = __builtin_bit_cast(uint2, h4);
    return make_uint4(l.x, l.y, h.x, h.y);
  };

  // L1 piece c of 8 for the tile at rows mt*32 of the buffer `ra` / `sa` point into, into register set P.
  auto l1_piece = [&](auto PC, int c, int mt) {
    constexpr int P = decltype(PC)::value;
    if constexpr (STAT_DPP) {
      if (c == 0) xs[P] = *reinterpret_cast<lds_f1>(static_cast<uintptr_t>(sa + mt * 128));
      if (c == 1) xd[P] = *reinterpret_cast<lds_f1>(static_cast<uintptr_t>(sa + BQ * 4 + mt * 128));
    } else if (c < 4) {
      const floatx4 x = *reinterpret_cast<lds_f4>(static_cast<uintptr_t>(sa + mt * 128 + c * 32));
      s[P][c * 4 + 0] = x.x; s[P][c * 4 + 1] = x.y; s[P][c * 4 + 2] = x.z; s[P][c * 4 + 3] = x.w;
    } else {
      const floatx4 x = *reinterpret_cast<lds_f4>(static_cast<uintptr_t>(sa + BQ * 4 + mt * 128 + (c - 4) * 32));
      dp[P][(c - 4) * 4 + 0] = x.x; dp[P][(c - 4) * 4 + 1] = x.y; dp[P][(c - 4) * 4 + 2] = x.z; dp[P][(c - 4) * 4 + 3] = x.w;
    }
    if (c % 2 == 0) qr[c / 2] = read16(ra[c / 2] + mt * 32 * tile_row_bytes<DP>());
    else dor[c / 2] = read16(ra[c / 2] + ROWS + mt * 32 * tile_row_bytes<DP>());
  };
  // MFMA c of 8 of stage A into register set P; FRESH: the accumulators start from zero.
  auto a_piece = [&](auto PC, auto FRESH, int c) {
    constexpr int P = decltype(PC)::value;
    constexpr bool Z = decltype(FRESH)::value;
    if (c % 2 == 0) s[P] = Mma<T>::run(qr[c / 2], kf[c / 2], (Z && c == 0) ? zero16() : s[P]);
    else dp[P] = Mma<T>::run(dor[c / 2], vf[c / 2], (Z && c == 1) ? zero16() : dp[P]);
  };
  // VALU piece C of 8 of stage B on register set P: elements 2C and 2C+1.
  auto b_piece = [&](auto PC, auto CC) {
    constexpr int P = decltype(PC)::value;
    constexpr int c = decltype(CC)::value;
    float s0 = s[P][2 * c], s1 = s[P][2 * c + 1], d0 = dp[P][2 * c], d1 = dp[P][2 * c + 1];
    if constexpr (STAT_DPP) {
      s0 += row_bcast<2 * c>(xs[P]);
      s1 += row_bcast<2 * c + 1>(xs[P]);
      d0 += row_bcast<2 * c>(xd[P]);
      d1 += row_bcast<2 * c + 1>(xd[P]);
    }
    const float p0 = fexp2(s0), p1 = fexp2(s1);
    pw[c] = Mma<T>::pack2(p0, p1);
    dw[c] = Mma<T>::pack2(p0 * d0, p1 * d1);
    // Pins the arithmetic here, under the MFMA issued just before it: without a use in this
    // block the compiler sinks it to the block after the barrier, where the results are read.
    asm volatile("" : "+v"(pw[c]), "+v"(dw[c]));
  };
  // L2 piece c of 4: the transposed fragments of 16 of the tile's rows for one 32-column block.
  auto l2_piece = [&](int c, int mt) {
    const int hf = c / 2, dt = c % 2;
    const int off = (mt * 2 + hf) * 16 * tile_row_bytes<DP>();
    tdo[hf][dt] = read_tr(tlo[dt] + ROWS + off, thi[dt] + ROWS + off);
    tq[hf][dt] = read_tr(tlo[dt] + off, thi[dt] + off);
  };
  // MFMA c of 8 of stage C.
  auto c_piece = [&](int c) {
    const int hf = c / 4, dt = (c % 4) / 2;
    if (c % 2 == 0) acc_v[dt] = Mma<T>::run(tdo[hf][dt], pf[hf], acc_v[dt]);
    else acc_k[dt] = Mma<T>::run(tq[hf][dt], dsf[hf], acc_k[dt]);
  };
  auto pack_frags = [&]() {
    pf[0] = make_uint4(pw[0], pw[1], pw[2], pw[3]);
    pf[1] = make_uint4(pw[4], pw[5], pw[6], pw[7]);
    dsf[0] = make_uint4(dw[0], dw[1], dw[2], dw[3]);
    dsf[1] = make_uint4(dw[4], dw[5], dw[6], dw[7]);
  };
  // Publishes the next step's buffer (its copies were issued a step ago) and starts the
  // copies of the step after it into the buffer that the previous step has finished with.
  // The barrier needs no wait for this wave's LDS reads: the ones still in flight (stage L2 of
  // the current tile) read the current step's buffer, not the one about to be overwritten.
  auto publish = [&]() {
    MG_ATTN_WAIT_VMCNT((kAttnRing - 3) * 5);  // all but the younger steps' copies
    asm volatile("s_barrier" ::: "memory");
  };
  // One iteration of the walk for tile g, whose S / dP are in register set P (= g % 2, the
  // tile's half of its step).  NEXT: tile g + 1 exists (stage A for it); NEXT2: tile g + 2
  // exists (stage L1 for it); FRESH: the accumulators of tile g + 1 start from zero (not from
  // the causal presets).
  auto iteration = [&](auto PC, auto NEXT, auto NEXT2, auto FRESH, int g) {
    constexpr int P = decltype(PC)::value;
    using PN = std::integral_constant<int, P ^ 1>;
    static_for<8>([&](auto CC) {
      constexpr int c = decltype(CC)::value;
      if (decltype(NEXT)::value) a_piece(PN{}, FRESH, c);
      b_piece(PC, CC);
      if (c >= 4) l2_piece(c - 4, P);
      __builtin_amdgcn_sched_barrier(0);
    });
    pack_frags();
    if (P == 0) publish();
    const int step2 = g / 2 + kAttnRing - 1;
    const int buf2 = step2 % kAttnRing;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      c_piece(c);
      if (decltype(NEXT2)::value) l1_piece(PC, c, P);
      if (P == 0 && c < 5) issue_piece(c, step2, buf2);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (P == 1) {
      advance_l1();
      advance_l2();
    }
  };

  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using Yes = std::true_type;
  using No = std::false_type;

#pragma unroll
  for (int st = 0; st < kAttnRing - 1; ++st) issue_step(st, st);
  MG_ATTN_WAIT_VMCNT((kAttnRing - 2) * 5);
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  // Causal: wave w's keys meet the diagonal in tile w of the walk.  It joins the walk at the
  // even tile gstart <= w (only the barriers and copies of the steps before that), with the
  // diagonal folded into the start values of the S accumulators of its first two tiles:
  // waves 0 and 2 mask the diagonal in their first tile; waves 1 and 3 see nothing in their
  // first tile and the diagonal in their second.
  const int gstart = CAUSAL ? min(wave_u & ~1, G) : 0;
  for (int g = 0; g < gstart; g += 2) {
    publish();
    issue_step(g / 2 + kAttnRing - 1, (g / 2 + kAttnRing - 1) % kAttnRing);
    advance_l1();
    advance_l2();
  }
  if (gstart < G) {
    const bool odd = CAUSAL && (wave_u & 1);
    // Stage L1 of the first two tiles; the S accumulators then start from 0 (or -lse) where
    // the key (column lane % 32) may see the query (row acc_row(r)) and from -inf where not.
    if (STAT_DPP) {
      s[0] = zero16(); s[1] = zero16(); dp[0] = zero16(); dp[1] = zero16();
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) l1_piece(P0{}, c, 0);
    if (CAUSAL) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[0][r] = (!odd && lane % 32 <= acc_row(r, lane)) ? s[0][r] : -INFINITY;
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) a_piece(P0{}, No{}, c);
#pragma unroll
    for (int c = 0; c < 8; ++c) l1_piece(P1{}, c, 1);
    if (CAUSAL) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[1][r] = (!odd || lane % 32 <= acc_row(r, lane)) ? s[1][r] : -INFINITY;
    }
    advance_l1();
    using Fresh = std::integral_constant<bool, STAT_DPP>;  // without STAT_DPP stage L1 sets the accumulators
    int g = gstart;
    if (g + 2 < G) {
      iteration(P0{}, Yes{}, Yes{}, No{}, g);
      iteration(P1{}, Yes{}, Yes{}, Fresh{}, g + 1);
      for (g += 2; g + 2 < G; g += 2) {
        iteration(P0{}, Yes{}, Yes{}, Fresh{}, g);
        iteration(P1{}, Yes{}, Yes{}, Fresh{}, g + 1);
      }
      iteration(P0{}, Yes{}, No{}, Fresh{}, g);
    } else {
      iteration(P0{}, Yes{}, No{}, No{}, g);
    }
    iteration(P1{}, No{}, No{}, Fresh{}, g + 1);
  }

  if (n < a.S) {
    T* outk = dk + qkv_at(a, b, n, h);
    T* outv = dv + qkv_at(a, b, n, h);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = dt * 32 + g * 8 + half * 4;
        if (d < a.D) {
          store4<T>(outk + d, acc_k[dt], g, scale);
          store4<T>(outv + d, acc_v[dt], g, 1.0f);
        }
      }
  }
}

// ---- dQ: software-pipelined walk (head dim <= 64, no bias) -------------------------------
// The same schedule as attn_dkdv_pipe_block with the roles exchanged: a wave keeps 32 queries
// (Q pre-scaled and dO as B operands, -lse and -delta as the lane-constant start values of the
// S^T and dP^T accumulators) and walks the keys in 32-key tiles, 64 keys per step through the
// ring of three buffers:
//   L1(g)  the eight row fragments of the K and V tile
//   A(g)   S^T = K Q^T - lse, dP^T = V dO^T - delta   (eight MFMAs)
//   B(g)   dS^T = exp2(S^T) dP^T, rounded and packed
//   L2(g)  the transposed fragments of the K tile
//   C(g)   dQ^T += K^T dS^T                             (four MFMAs)
// The keys are walked from the last step down to the first.  The only tiles that need a mask
// (keys past the end of the sequence; causal: keys after the query) are then in the first step
// a wave takes part in, where the mask goes into the start values of the S^T accumulators of
// its first two tiles; every later tile is unmasked.  Causal: a wave joins the walk at the
// step that holds its last visible key.

template <int DP>
constexpr int dq_pipe_buf_bytes() {
  return 2 * 64 * tile_row_bytes<DP>();  // a K tile and a V tile of 64 keys
}
template <int DP>
constexpr int dq_pipe_lds_bytes() {
  return kAttnRing * dq_pipe_buf_bytes<DP>();
}

template <typename T, int DP, bool CAUSAL>
__device__ __forceinline__ void attn_dq_pipe_block(const int block, char* smem, const T* __restrict__ d_o,
                                                   const T* __restrict__ q, const T* __restrict__ k,
                                                   const T* __restrict__ v, const float* __restrict__ lse,
                                                   const float* __restrict__ delta, T* __restrict__ dq,
                                                   const AttnDims& a, float scale) {
  static_assert(DP == 64, "tile shapes below are written for a 64-wide head");
  constexpr int BM = 128, BN = 64, KS = DP / 16, DT = DP / 32;
  constexpr int ROWS = BN * tile_row_bytes<DP>();
  constexpr int BUF = dq_pipe_buf_bytes<DP>();

  const int nqb = (a.S + BM - 1) / BM;
  const int n_bh = a.B * a.H;
  const int qb = CAUSAL ? nqb - 1 - block / n_bh : block / n_bh;  // heaviest query blocks first
  const int h = (block % n_bh) % a.H;
  const int b = (block % n_bh) / a.H;
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int half = lane / 32;
  const TileLane16<DP> at(lane);
  const int m_wave = qb * BM + wave_u * 32;
  const int m = m_wave + lane % 32;
  const int64_t bh = static_cast<int64_t>(b) * a.H + h;

  const float c = scale * kAttnLog2e;
  uint4 qf[KS], dof[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 16 + half * 8;
    const bool ok = m < a.S && d < a.D;
    qf[ks] = ok ? *reinterpret_cast<const uint4*>(q + qkv_at(a, b, m, h) + d) : make_uint4(0, 0, 0, 0);
    qf[ks] = scale_frag<T>(qf[ks], c);
    dof[ks] = ok ? *reinterpret_cast<const uint4*>(d_o + o_at(a, b, h, m) + d) : make_uint4(0, 0, 0, 0);
  }
  // Rows past the end get lse = +inf so that their probabilities vanish.
  const float nlse2 = m < a.S ? -lse[bh * a.S + m] * kAttnLog2e : -INFINITY;
  const float ndl = m < a.S ? -delta[bh * a.S + m] : 0.f;
  const floatx16 s_init = splat16(nlse2), dp_init = splat16(ndl);
  floatx16 acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) acc[dt] = zero16();

  // Keys [0, n_end) in steps of 64, walked downwards: step i covers keys n_top - 64 (i + 1) ..
  const int n_end = CAUSAL ? min(a.S, qb * BM + BM) : a.S;
  const int nsteps = (n_end + BN - 1) / BN;
  const int G = 2 * nsteps;
  auto step_key0 = [&](int step) { return (nsteps - 1 - step) * BN; };

  // ---- copies: step i -> buffer i % kAttnRing (see attn_dkdv_pipe_block) ----
  const int cp_row = lane / 8;
  const int cp_chunk = (lane % 8) ^ tile_swz16(8 * (wave % 2) + cp_row);
  const unsigned cp_col_bytes = cp_chunk * 8 < a.D ? cp_chunk * 16 : 0;
  const char* k_bh = reinterpret_cast<const char*>(k + qkv_at(a, b, 0, h));
  const char* v_bh = reinterpret_cast<const char*>(v + qkv_at(a, b, 0, h));
  const unsigned pitch = static_cast<unsigned>(a.ld) * 2;
  const unsigned smem_base = lds_address(smem);
  // Copy c of 4 of step `step` (clamped to the walk's last step) into buffer `buf`: K rows, V
  // rows, K rows, V rows.  Keys past the end of the sequence copy its last row.
  auto issue_piece = [&](int c, int step, int buf) {
    const int n0 = step_key0(min(step, nsteps - 1));
    const int jj = c / 2;
    const bool is_v = c % 2;
    const int j = wave_u + 4 * jj;
    const int row = min(8 * j + cp_row, a.S - 1 - n0);
    const char* rows0 = (is_v ? v_bh : k_bh) + static_cast<int64_t>(n0) * pitch;
    const unsigned dst = __builtin_amdgcn_readfirstlane(smem_base + buf * BUF + (is_v ? ROWS : 0) + j * 1024);
    const unsigned off = row * pitch + cp_col_bytes;
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(rows0) : "memory");
  };
  auto issue_step = [&](int step, int buf) {
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) issue_piece(cc, step, buf);
  };

  // ---- stages ----
  floatx16 s[2], dp[2];
  uint4 kr[KS], vr[KS], kt[2][DT], dsf[2];
  uint32_t dw[8];
  typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
  using lds_u4 = __attribute__((address_space(3))) const uintx4*;
  using lds_i16x4 = __attribute__((address_space(3))) short4_t*;
  unsigned ra[KS], tlo[DT], thi[DT];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) ra[ks] = smem_base + at.rows[ks];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    tlo[dt] = smem_base + at.tr_lo[dt];
    thi[dt] = smem_base + at.tr_hi[dt];
  }
  int buf_l1 = 0, buf_l2 = 0;
  auto advance_l1 = [&]() {
    const int d = buf_l1 == kAttnRing - 1 ? -(kAttnRing - 1) * BUF : BUF;
    buf_l1 = buf_l1 == kAttnRing - 1 ? 0 : buf_l1 + 1;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ra[ks] += d;
  };
  auto advance_l2 = [&]() {
    const int d = buf_l2 == kAttnRing - 1 ? -(kAttnRing - 1) * BUF : BUF;
    buf_l2 = buf_l2 == kAttnRing - 1 ? 0 : buf_l2 + 1;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      tlo[dt] += d;
      thi[dt] += d;
    }
  };
  auto read16 = [](unsigned addr) {
    const uintx4 x = *reinterpret_cast<lds_u4>(static_cast<uintptr_t>(addr));
    return make_uint4(x[0], x[1], x[2], x[3]);
  };
  auto read_tr = [](unsigned lo, unsigned hi) {
    const short4_t l4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_i16x4>(static_cast<uintptr_t>(lo)));
    const short4_t h4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_i16x4>(static_cast<uintptr_t>(hi)));
    const uint2 l = __builtin_bit_cast(uint2, l4), h2 = __builtin_bit_cast(uint2, h4);
    return make_uint4(l.x, l.y, h2.x, h2.y);
  };
  // L1 piece cc of 8 for the tile at rows mt*32 of the buffer `ra` points into.
  auto l1_piece = [&](int cc, int mt) {
    if (cc % 2 == 0) kr[cc / 2] = read16(ra[cc / 2] + mt * 32 * tile_row_bytes<DP>());
    else vr[cc / 2] = read16(ra[cc / 2] + ROWS + mt * 32 * tile_row_bytes<DP>());
  };
  // MFMA cc of 8 of stage A into register set P; FRESH: start from -lse / -delta (not from the presets).
  auto a_piece = [&](auto PC, auto FRESH, int cc) {
    constexpr int P = decltype(PC)::value;
    constexpr bool Z = decltype(FRESH)::value;
    if (cc % 2 == 0) s[P] = Mma<T>::run(kr[cc / 2], qf[cc / 2], (Z && cc == 0) ? s_init : s[P]);
    else dp[P] = Mma<T>::run(vr[cc / 2], dof[cc / 2], (Z && cc == 1) ? dp_init : dp[P]);
  };
  // VALU piece cc of 8 of stage B on register set P: elements 2cc and 2cc+1.
  auto b_piece = [&](auto PC, int cc) {
    constexpr int P = decltype(PC)::value;
    const float p0 = fexp2(s[P][2 * cc]), p1 = fexp2(s[P][2 * cc + 1]);
    dw[cc] = Mma<T>::pack2(p0 * dp[P][2 * cc], p1 * dp[P][2 * cc + 1]);
    asm volatile("" : "+v"(dw[cc]));  // keeps the arithmetic under the MFMA issued before it
  };
  // L2 piece cc of 4: the transposed fragment of 16 of the K tile's rows for one 32-column block.
  auto l2_piece = [&](int cc, int mt) {
    const int hf = cc / 2, dt = cc % 2;
    const int off = (mt * 2 + hf) * 16 * tile_row_bytes<DP>();
    kt[hf][dt] = read_tr(tlo[dt] + off, thi[dt] + off);
  };
  // MFMA cc of 4 of stage C.
  auto c_piece = [&](int cc) {
    const int hf = cc / 2, dt = cc % 2;
    acc[dt] = Mma<T>::run(kt[hf][dt], dsf[hf], acc[dt]);
  };
  auto publish = [&]() {
    MG_ATTN_WAIT_VMCNT((kAttnRing - 3) * 4);  // all but the younger steps' copies
    asm volatile("s_barrier" ::: "memory");
  };
  auto iteration = [&](auto PC, auto NEXT, auto NEXT2, auto FRESH, int g) {
    constexpr int P = decltype(PC)::value;
    using PN = std::integral_constant<int, P ^ 1>;
#pragma unroll
    for (int cc = 0; cc < 8; ++cc) {
      if (decltype(NEXT)::value) a_piece(PN{}, FRESH, cc);
      b_piece(PC, cc);
      if (cc >= 4) l2_piece(cc - 4, P);
      __builtin_amdgcn_sched_barrier(0);
    }
    dsf[0] = make_uint4(dw[0], dw[1], dw[2], dw[3]);
    dsf[1] = make_uint4(dw[4], dw[5], dw[6], dw[7]);
    if (P == 0) publish();
    const int step2 = g / 2 + kAttnRing - 1;
    const int buf2 = step2 % kAttnRing;
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      c_piece(cc);
      if (decltype(NEXT2)::value) {
        l1_piece(2 * cc, P);
        l1_piece(2 * cc + 1, P);
      }
      if (P == 0) issue_piece(cc, step2, buf2);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (P == 1) {
      advance_l1();
      advance_l2();
    }
  };

  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using Yes = std::true_type;
  using No = std::false_type;

#pragma unroll
  for (int st = 0; st < kAttnRing - 1; ++st) issue_step(st, st);
  MG_ATTN_WAIT_VMCNT((kAttnRing - 2) * 4);
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  // Causal: the wave joins at the step that holds its last visible key, m_wave + 31.
  const int first_step = CAUSAL ? max(0, nsteps - 1 - (m_wave + 31) / BN) : 0;
  const int gstart = min(2 * first_step, G);
  for (int g = 0; g < gstart; g += 2) {
    publish();
    issue_step(g / 2 + kAttnRing - 1, (g / 2 + kAttnRing - 1) % kAttnRing);
    advance_l1();
    advance_l2();
  }
  if (gstart < G) {
    // The first two tiles: S^T accumulator r of tile t stands for key n0 + 32 t + acc_row(r); it
    // starts from -lse if that key exists and (causal) does not come after this lane's query.
    const int n0 = step_key0(gstart / 2);
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = n0 + 32 * t + acc_row(r, lane);
        const bool ok = key < a.S && (!CAUSAL || key <= m);
        s[t][r] = ok ? nlse2 : -INFINITY;
      }
    dp[0] = dp_init;
    dp[1] = dp_init;
#pragma unroll
    for (int cc = 0; cc < 8; ++cc) l1_piece(cc, 0);
#pragma unroll
    for (int cc = 0; cc < 8; ++cc) a_piece(P0{}, No{}, cc);
#pragma unroll
    for (int cc = 0; cc < 8; ++cc) l1_piece(cc, 1);
    advance_l1();
    int g = gstart;
    if (g + 2 < G) {
      iteration(P0{}, Yes{}, Yes{}, No{}, g);
      iteration(P1{}, Yes{}, Yes{}, Yes{}, g + 1);
      for (g += 2; g + 2 < G; g += 2) {
        iteration(P0{}, Yes{}, Yes{}, Yes{}, g);
        iteration(P1{}, Yes{}, Yes{}, Yes{}, g + 1);
      }
      iteration(P0{}, Yes{}, No{}, Yes{}, g);
    } else {
      iteration(P0{}, Yes{}, No{}, No{}, g);
    }
    iteration(P1{}, No{}, No{}, Yes{}, g + 1);
  }

  if (m < a.S) {
    T* out = dq + qkv_at(a, b, m, h);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int d = dt * 32 + g4 * 8 + half * 4;
        if (d < a.D) store4<T>(out + d, acc[dt], g4, scale);
      }
  }
}

// ---- backward launches --------------------------------------------------------------------

// ---- whole heads in LDS (sequences up to 256, head dim 64, no bias) -----------------------
// At short sequences the walks above are all prologue: a workgroup runs two to four steps
// after loading its resident operand and filling its ring, four workgroups per (batch, head)
// each read Q, K, V and dO again, and delta needs a launch of its own.  But the four tensors
// of one (batch, head) are then at most 4 x 256 x 128 bytes = 128 KB and fit one CU's LDS.
// Here one workgroup of eight waves copies them in once (global_load_lds, the conflict-free
// image of the pipelined walks), computes delta = rowsum(dO o O) itself, and after one barrier
// every wave runs, straight from LDS, first the dK/dV products of its own 32 keys over the
// query tiles and then the dQ products of its own 32 queries over the key tiles: the per-tile
// arithmetic of attn_dkdv_block and attn_dq_block, with no streaming and no further barrier.
// Causal: wave w meets 8 - w query tiles in the first pass and w + 1 key tiles in the second,
// so the waves carry equal loads without waiting for each other between the passes.
constexpr int kResidentS = 256;
constexpr int kResidentTensor = kResidentS * 128;                        // bytes of one tensor's image
constexpr int kResidentLds = 4 * kResidentTensor + 2 * kResidentS * 4;   // Q, K, V, dO, -lse, -delta

template <typename T, bool CAUSAL>
__global__ __launch_bounds__(512, 1) void attn_bwd_resident_kernel(
    const T* __restrict__ d_o, const T* __restrict__ o, const T* __restrict__ q, const T* __restrict__ k,
    const T* __restrict__ v, const float* __restrict__ lse, T* __restrict__ dq, T* __restrict__ dk, T* __restrict__ dv,
    AttnDims a, float scale) {
  constexpr int DP = 64, KS = DP / 16, DT = DP / 32;
  __shared__ __attribute__((aligned(1024))) char smem[kResidentLds];
  const char* const q_rows = smem;
  const char* const k_rows = smem + kResidentTensor;
  const char* const v_rows = smem + 2 * kResidentTensor;
  const char* const do_rows = smem + 3 * kResidentTensor;
  float* const nlse_s = reinterpret_cast<float*>(smem + 4 * kResidentTensor);
  float* const ndelta_s = nlse_s + kResidentS;

  const int bh = blockIdx.x;
  const int b = bh / a.H, h = bh % a.H;
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int half = lane / 32;
  const int n_tiles = (a.S + 31) / 32;

  // ---- copies: wave instruction j of a tensor covers its rows 8j .. 8j+7 (1 KB); this wave
  // issues j = wave, wave + 8, ...  Lane l writes chunk position l % 8 of row 8j + l / 8 and
  // therefore names the source chunk (l % 8) ^ swz16(row), with row % 16 = 8 (wave % 2) + l / 8.
  // Rows past the end of the sequence (up to the end of its last 32-row tile) copy the last row.
  {
    const unsigned smem_base = lds_address(smem);
    const int cp_row = lane / 8;
    const unsigned cp_col = static_cast<unsigned>(((lane % 8) ^ tile_swz16(8 * (wave % 2) + cp_row)) * 16);
    const unsigned qkv_pitch = static_cast<unsigned>(a.ld) * 2, do_pitch = static_cast<unsigned>(o_ld(a)) * 2;
    const char* const src[4] = {reinterpret_cast<const char*>(q + qkv_at(a, b, 0, h)),
                                reinterpret_cast<const char*>(k + qkv_at(a, b, 0, h)),
                                reinterpret_cast<const char*>(v + qkv_at(a, b, 0, h)),
                                reinterpret_cast<const char*>(d_o + o_at(a, b, h, 0))};
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int jj = 0; jj < kResidentS / 64; ++jj) {
        const int j = wave + 8 * jj;
        if (8 * j < n_tiles * 32) {
          const int row = min(8 * j + cp_row, a.S - 1);
          const unsigned off = row * (t == 3 ? do_pitch : qkv_pitch) + cp_col;
          const unsigned dst = __builtin_amdgcn_readfirstlane(smem_base + t * kResidentTensor + j * 1024);
          asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(src[t]) : "memory");
        }
      }
  }
  // ---- delta and the statistics: two threads per row, 32 columns each; O comes from global
  // memory, dO from its LDS image once the copies have landed.  Stored negated, lse in log2
  // units: they start the accumulators of the S and dP products.  Rows past the end carry
  // -lse = -inf (their probabilities vanish) and delta = 0.
  {
    const int i = threadIdx.x / 2, part = threadIdx.x % 2;
    const int ic = min(i, a.S - 1);
    uint4 ow[4];
    const T* orow = o + o_at(a, b, h, ic) + part * 32;
#pragma unroll
    for (int c = 0; c < 4; ++c) ow[c] = *reinterpret_cast<const uint4*>(orow + 8 * c);
    const float nl = i < a.S ? -lse[static_cast<int64_t>(bh) * a.S + i] * kAttnLog2e : -INFINITY;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's copies have landed
    __syncthreads();
    float dot = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      float x[8], y[8];
      VecIO<T, 8>::load(reinterpret_cast<const T*>(&ow[c]), x);
      VecIO<T, 8>::load(reinterpret_cast<const T*>(do_rows + tile16_chunk_at<DP>(i, part * 4 + c)), y);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot = fmaf(x[e], y[e], dot);
    }
    dot += dpp_move<kDppQuadXor1>(dot);
    if (part == 0) {
      nlse_s[i] = nl;
      ndelta_s[i] = i < a.S ? -dot : 0.f;
    }
  }
  __syncthreads();

  const TileLane16<DP> at(lane);
  const float c = scale * kAttnLog2e;
  if (wave >= n_tiles) return;  // no keys and no queries for this wave

  // ---- pass 1: dK, dV of keys 32 wave .. 32 wave + 31
  {
    const int n_wave = wave * 32;
    const int n = n_wave + lane % 32;
    uint4 kf[KS], vf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[ks] = scale_frag<T>(frag_rows<DP>(k_rows, at, wave, ks), c);
      vf[ks] = frag_rows<DP>(v_rows, at, wave, ks);
    }
    floatx16 acc_k[DT], acc_v[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      acc_k[dt] = zero16();
      acc_v[dt] = zero16();
    }
    for (int mt = CAUSAL ? wave : 0; mt < n_tiles; ++mt) {
      const int m0 = mt * 32;
      const bool plain = n_wave + 31 < a.S && (!CAUSAL || mt > wave);
      floatx16 s, dp;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float4 l4 = *reinterpret_cast<const float4*>(&nlse_s[m0 + g * 8 + half * 4]);
        const float4 d4 = *reinterpret_cast<const float4*>(&ndelta_s[m0 + g * 8 + half * 4]);
        s[g * 4 + 0] = l4.x; s[g * 4 + 1] = l4.y; s[g * 4 + 2] = l4.z; s[g * 4 + 3] = l4.w;
        dp[g * 4 + 0] = d4.x; dp[g * 4 + 1] = d4.y; dp[g * 4 + 2] = d4.z; dp[g * 4 + 3] = d4.w;
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        s = Mma<T>::run(frag_rows<DP>(q_rows, at, mt, ks), kf[ks], s);
        dp = Mma<T>::run(frag_rows<DP>(do_rows, at, mt, ks), vf[ks], dp);
      }
      uint4 tq[2][DT], tdo[2][DT];
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          tdo[hf][dt] = frag_transposed<DP>(do_rows, at, dt, mt * 2 + hf);
          tq[hf][dt] = frag_transposed<DP>(q_rows, at, dt, mt * 2 + hf);
        }
      __builtin_amdgcn_sched_barrier(0);
      if (plain) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fexp2(s[r]);
          s[r] = p;
          dp[r] = p * dp[r];
        }
      } else {
        const bool col_ok = n < a.S;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          bool valid = col_ok;
          if (CAUSAL) valid = valid && n <= m0 + acc_row(r, lane);
          float p = fexp2(s[r]);  // rows past the end started from -inf: p = 0
          p = valid ? p : 0.f;
          s[r] = p;
          dp[r] = p * dp[r];
        }
      }
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const uint4 pf = frag_from_acc<T>(s, hf);
        const uint4 dsf = frag_from_acc<T>(dp, hf);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          acc_v[dt] = Mma<T>::run(tdo[hf][dt], pf, acc_v[dt]);
          acc_k[dt] = Mma<T>::run(tq[hf][dt], dsf, acc_k[dt]);
        }
      }
    }
    if (n < a.S) {
      T* outk = dk + qkv_at(a, b, n, h);
      T* outv = dv + qkv_at(a, b, n, h);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int d = dt * 32 + g * 8 + half * 4;
          store4<T>(outk + d, acc_k[dt], g, scale);
          store4<T>(outv + d, acc_v[dt], g, 1.0f);
        }
    }
  }

  // ---- pass 2: dQ of queries 32 wave .. 32 wave + 31
  {
    const int m_wave = wave * 32;
    const int m = m_wave + lane % 32;
    uint4 qf[KS], dof[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = scale_frag<T>(frag_rows<DP>(q_rows, at, wave, ks), c);
      dof[ks] = frag_rows<DP>(do_rows, at, wave, ks);
    }
    const floatx16 s_init = splat16(nlse_s[m]), dp_init = splat16(ndelta_s[m]);
    floatx16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = zero16();
    const int nt_end = CAUSAL ? wave + 1 : n_tiles;
    for (int nt = 0; nt < nt_end; ++nt) {
      const int nb = nt * 32;
      floatx16 s = s_init, dp = dp_init;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        s = Mma<T>::run(frag_rows<DP>(k_rows, at, nt, ks), qf[ks], s);
        dp = Mma<T>::run(frag_rows<DP>(v_rows, at, nt, ks), dof[ks], dp);
      }
      uint4 kt[2][DT];
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) kt[hf][dt] = frag_transposed<DP>(k_rows, at, dt, nt * 2 + hf);
      __builtin_amdgcn_sched_barrier(0);
      const bool plain = nb + 32 <= a.S && (!CAUSAL || nt < wave);
      if (plain) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = fexp2(s[r]) * dp[r];
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int n = nb + acc_row(r, lane);
          bool valid = n < a.S;
          if (CAUSAL) valid = valid && n <= m;
          float p = fexp2(s[r]);
          p = valid ? p : 0.f;
          s[r] = p * dp[r];  // dS^T
        }
      }
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const uint4 dsf = frag_from_acc<T>(s, hf);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[dt] = Mma<T>::run(kt[hf][dt], dsf, acc[dt]);
      }
    }
    if (m < a.S) {
      T* out = dq + qkv_at(a, b, m, h);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) store4<T>(out + dt * 32 + g * 8 + half * 4, acc[dt], g, scale);
    }
  }
}

template <typename T, int DP, int MQ, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(kAttnThreads, DP <= 128 ? 2 : 1) void attn_dq_mfma_kernel(const T* __restrict__ d_o, const T* __restrict__ q,
                                                                       const T* __restrict__ k, const T* __restrict__ v,
                                                                       const T* __restrict__ mask,
                                                                       const float* __restrict__ lse,
                                                                       const float* __restrict__ delta,
                                                                       T* __restrict__ dq, AttnDims a, float scale) {
  __shared__ __attribute__((aligned(16))) char smem[dq_lds_bytes<DP>()];
  if constexpr (DP <= 128) {
    attn_dq_block<T, DP, MQ, CAUSAL, HAS_BIAS>(blockIdx.x, smem, d_o, q, k, v, mask, lse, delta, dq, a, scale);
  } else {
    // wider heads: each half of the head dimension of a query block is a workgroup of its own
    const int block = blockIdx.x / kAttnWideSplit;
    if (blockIdx.x % kAttnWideSplit == 0)
      attn_dq_block<T, DP, MQ, CAUSAL, HAS_BIAS, kAttnWideSplit, 0>(block, smem, d_o, q, k, v, mask, lse, delta, dq, a, scale);
    else
      attn_dq_block<T, DP, MQ, CAUSAL, HAS_BIAS, kAttnWideSplit, 1>(block, smem, d_o, q, k, v, mask, lse, delta, dq, a, scale);
  }
}

template <typename T, int DP, bool CAUSAL>
__global__ __launch_bounds__(kAttnThreads, 2) void attn_dq_pipe_kernel(const T* __restrict__ d_o, const T* __restrict__ q,
                                                                       const T* __restrict__ k, const T* __restrict__ v,
                                                                       const float* __restrict__ lse,
                                                                       const float* __restrict__ delta,
                                                                       T* __restrict__ dq, AttnDims a, float scale) {
  __shared__ __attribute__((aligned(1024))) char smem[dq_pipe_lds_bytes<DP>()];
  attn_dq_pipe_block<T, DP, CAUSAL>(blockIdx.x, smem, d_o, q, k, v, lse, delta, dq, a, scale);
}

// The pipelined walk with a launch of its own.
template <typename T, int DP, bool CAUSAL>
__global__ __launch_bounds__(kAttnThreads, 2) void attn_dkdv_pipe_kernel(
    const T* __restrict__ d_o, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const float* __restrict__ nlse, const float* __restrict__ ndelta, int s_pad, T* __restrict__ dk, T* __restrict__ dv,
    AttnDims a, float scale) {
  __shared__ __attribute__((aligned(1024))) char smem[dkdv_pipe_lds_bytes<DP>()];
  attn_dkdv_pipe_block<T, DP, CAUSAL, kAttnStatDpp>(blockIdx.x, smem, d_o, q, k, v, nlse, ndelta, s_pad, dk, dv, a, scale);
}

template <typename T, int DP, bool CAUSAL, bool HAS_BIAS>
__global__ __launch_bounds__(kAttnThreads, DP <= 64 ? 2 : 1) void attn_dkdv_mfma_kernel(
    const T* __restrict__ d_o, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const T* __restrict__ mask, const float* __restrict__ lse, const float* __restrict__ delta, T* __restrict__ dk,
    T* __restrict__ dv, AttnDims a, float scale) {
  __shared__ __attribute__((aligned(16))) char smem[dkdv_lds_bytes<DP, dkdv_long_step<DP>()>()];
  if constexpr (DP <= 128) {
    attn_dkdv_block<T, DP, dkdv_long_step<DP>(), CAUSAL, HAS_BIAS>(blockIdx.x, smem, d_o, q, k, v, mask, lse, delta, dk, dv, a, scale);
  } else {
    const int block = blockIdx.x / kAttnWideSplit;
    if (blockIdx.x % kAttnWideSplit == 0)
      attn_dkdv_block<T, DP, 32, CAUSAL, HAS_BIAS, kAttnWideSplit, 0>(block, smem, d_o, q, k, v, mask, lse, delta, dk, dv, a, scale);
    else
      attn_dkdv_block<T, DP, 32, CAUSAL, HAS_BIAS, kAttnWideSplit, 1>(block, smem, d_o, q, k, v, mask, lse, delta, dk, dv, a, scale);
  }
}

// Both walks in one launch (head dims up to 64, where the two have the same occupancy):
// groups of eight consecutive workgroups alternate between dK/dV and dQ blocks, so every
// XCD runs both kinds, and short sequences pay for one launch instead of two.  `blocks` is
// the block count of each walk; the grid is 2 * round_up(blocks, 8) workgroups.
template <typename T, int DP, bool CAUSAL, bool HAS_BIAS, bool PIPE>
__global__ __launch_bounds__(kAttnThreads, 2) void attn_bwd_mfma_kernel(
    const T* __restrict__ d_o, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const T* __restrict__ mask, const float* __restrict__ lse, const float* __restrict__ delta, T* __restrict__ dq,
    T* __restrict__ dk, T* __restrict__ dv, AttnDims a, float scale, int blocks, const float* __restrict__ nlse,
    const float* __restrict__ ndelta, int s_pad) {
  constexpr int DKDV = PIPE ? dkdv_pipe_lds_bytes<DP>() : dkdv_lds_bytes<DP, 64>();
  constexpr int LDS = DKDV > dq_lds_bytes<DP>() ? DKDV : dq_lds_bytes<DP>();
  __shared__ __attribute__((aligned(1024))) char smem[LDS];
  const int block = (blockIdx.x / 16) * 8 + blockIdx.x % 8;
  if (block >= blocks) return;
  if ((blockIdx.x / 8) % 2 == 0) {
    if constexpr (PIPE)
      attn_dkdv_pipe_block<T, DP, CAUSAL, kAttnStatDpp>(block, smem, d_o, q, k, v, nlse, ndelta, s_pad, dk, dv, a, scale);
    else
      attn_dkdv_block<T, DP, 64, CAUSAL, HAS_BIAS>(block, smem, d_o, q, k, v, mask, lse, delta, dk, dv, a, scale);
  } else {
    if constexpr (PIPE)
      attn_dq_pipe_block<T, DP, CAUSAL>(block, smem, d_o, q, k, v, lse, delta, dq, a, scale);
    else
      attn_dq_block<T, DP, 1, CAUSAL, HAS_BIAS>(block, smem, d_o, q, k, v, mask, lse, delta, dq, a, scale);
  }
}

// ---- host side ---------------------------------------------------------------------------

bool attn_mfma_supported(int dtype, int64_t D, const void* const* ptrs, int nptrs) {
  if (dtype != MG_F16 && dtype != MG_BF16) return false;
  if (D % 8 != 0 || D > 256) return false;  // rows are read 16 bytes at a time
  for (int i = 0; i < nptrs; ++i)
    if (ptrs[i] != nullptr && !aligned16(ptrs[i])) return false;
  const char* force = env_str("MOGRAD_HIP_ATTN_GENERIC");
  if (force && force[0] == '1') return false;
  return true;
}

template <typename T, int DP>
static int fwd_typed(const void* q, const void* k, const void* v, const void* mask, void* o, float* lse, AttnDims a,
                     float scale, bool causal, bool has_bias, hipStream_t stream) {
  const int64_t blocks = static_cast<int64_t>(a.B) * a.H * ceil_div(a.S, 128);
#define MG_LAUNCH(C_, B_)                                                                                             \
  hipLaunchKernelGGL((attn_fwd_mfma_kernel<T, DP, C_, B_>), dim3(static_cast<unsigned>(blocks)), dim3(kAttnThreads), 0, \
                     stream, static_cast<const T*>(q), static_cast<const T*>(k), static_cast<const T*>(v),            \
                     static_cast<const T*>(mask), static_cast<T*>(o), lse, a, scale)
  if (causal) MG_LAUNCH(true, false);
  else if (has_bias) MG_LAUNCH(false, true);
  else MG_LAUNCH(false, false);
#undef MG_LAUNCH
  MG_LAUNCH_CHECK();
  return MG_OK;
}

// delta[row] = sum_d dO[row, d] * O[row, d] for contiguous rows of D = 8 * CPR elements, CPR a
// power of two: one 16-byte chunk of each tensor per thread, then a sum over the CPR
// neighbouring lanes that share a row.
template <typename T, int CPR>
__global__ __launch_bounds__(256) void attn_delta_rows_kernel(const T* __restrict__ d_o, const T* __restrict__ o,
                                                              float* __restrict__ delta, int64_t rows, int S, int H,
                                                              int o_bshd, AttnPaddedStats ps) {
  const int64_t chunk = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t row = chunk / CPR;
  float acc = 0.f;
  if (row < rows) {
    float x[8], y[8];
    VecIO<T, 8>::load(d_o + chunk * 8, x);
    VecIO<T, 8>::load(o + chunk * 8, y);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc = fmaf(x[e], y[e], acc);
  }
#pragma unroll
  for (int w = 1; w < CPR; w *= 2) acc += __shfl_xor(acc, w);
  if (row < rows && threadIdx.x % CPR == 0) {
    const int64_t idx = o_row_to_bhs(row, S, H, o_bshd);
    delta[idx] = acc;
    write_padded_stats(ps, idx, S, acc);
  }
}

template <typename T>
static int launch_delta(const T* d_o, const T* o, float* delta, int64_t rows, const AttnDims& a, hipStream_t stream,
                        AttnPaddedStats ps = {}) {
  const int D = a.D;
  const int cpr = D / 8;
  const bool vec = D % 8 == 0 && (cpr & (cpr - 1)) == 0 && cpr <= 16;
  if (vec) {
    const dim3 grid(static_cast<unsigned>(ceil_div(rows * cpr, 256)));
#define MG_DELTA(CPR_)                                                                                              \
  hipLaunchKernelGGL((attn_delta_rows_kernel<T, CPR_>), grid, dim3(256), 0, stream, d_o, o, delta, rows, a.S, a.H, \
                     a.o_bshd, ps)
    switch (cpr) {
      case 1: MG_DELTA(1); break;
      case 2: MG_DELTA(2); break;
      case 4: MG_DELTA(4); break;
      case 8: MG_DELTA(8); break;
      default: MG_DELTA(16); break;
    }
#undef MG_DELTA
  } else {
    hipLaunchKernelGGL((attn_delta_kernel<T>), dim3(static_cast<unsigned>(ceil_div(rows, 4))), dim3(256), 0, stream, d_o,
                       o, delta, rows, D, a.S, a.H, a.o_bshd, ps);
  }
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T, int DP>
static int bwd_typed(const void* d_o, const void* o, const void* q, const void* k, const void* v, const void* mask,
                     const float* lse, void* dq, void* dk, void* dv, AttnDims a, float scale, bool causal, bool has_bias,
                     hipStream_t stream) {
  const int64_t rows = static_cast<int64_t>(a.B) * a.H * a.S;
  // Short sequences of 64-wide heads: one workgroup per (batch, head) with the whole head in
  // LDS (attn_bwd_resident_kernel); no delta launch, no scratch.
  if constexpr (DP == 64) {
    if (a.D == 64 && a.S <= kResidentS && !has_bias && env_int("MOGRAD_HIP_ATTN_RESIDENT", 1) != 0 &&
        static_cast<int64_t>(a.S) * a.ld * 2 < 0x7fffffffLL) {
      const dim3 grid(static_cast<unsigned>(a.B * a.H));
      if (causal)
        hipLaunchKernelGGL((attn_bwd_resident_kernel<T, true>), grid, dim3(512), 0, stream, static_cast<const T*>(d_o),
                           static_cast<const T*>(o), static_cast<const T*>(q), static_cast<const T*>(k),
                           static_cast<const T*>(v), lse, static_cast<T*>(dq), static_cast<T*>(dk), static_cast<T*>(dv), a,
                           scale);
      else
        hipLaunchKernelGGL((attn_bwd_resident_kernel<T, false>), grid, dim3(512), 0, stream, static_cast<const T*>(d_o),
                           static_cast<const T*>(o), static_cast<const T*>(q), static_cast<const T*>(k),
                           static_cast<const T*>(v), lse, static_cast<T*>(dq), static_cast<T*>(dk), static_cast<T*>(dv), a,
                           scale);
      MG_LAUNCH_CHECK();
      return MG_OK;
    }
  }
  // The pipelined dK/dV walk (head dims up to 64, no bias) reads the row statistics negated
  // and padded per (batch, head) to a multiple of 64 rows; the delta kernel writes both forms.
  const bool pipe = DP <= 64 && !has_bias && env_int("MOGRAD_HIP_ATTN_DKDV_PIPE", 1) != 0;
  const int s_pad = static_cast<int>(ceil_div(a.S, 64) * 64);
  const int64_t padded = pipe ? static_cast<int64_t>(a.B) * a.H * s_pad : 0;
  Scratch delta;
  MG_TRY(delta.take((rows + 2 * padded) * static_cast<int64_t>(sizeof(float))));
  AttnPaddedStats ps;
  if (pipe) {
    ps.lse = lse;
    ps.nlse = delta.as<float>() + rows;
    ps.ndelta = ps.nlse + padded;
    ps.s_pad = s_pad;
  }
  MG_TRY(launch_delta(static_cast<const T*>(d_o), static_cast<const T*>(o), delta.as<float>(), rows, a, stream, ps));
  const int64_t blocks = static_cast<int64_t>(a.B) * a.H * ceil_div(a.S, 128);
  // One launch for both walks up to this sequence length.  Measured at 8192 tokens per batch of
  // twelve heads: causal, where the short walks of one kind fill the gaps the other leaves, 6-10 %
  // faster up to 2048 tokens and even at 4096; non-causal 4-6 % faster at 512 and 3-6 % slower
  // from 1024 on, where the two walks compete for the same CU.  MOGRAD_HIP_ATTN_FUSED_BWD_MAX_S
  // overrides it; 0 always launches dK/dV and dQ separately.
  const int fused_max_s = env_int("MOGRAD_HIP_ATTN_FUSED_BWD_MAX_S", causal ? 2048 : 512);
  const bool fused = DP <= 64 && a.S <= fused_max_s && 2 * (blocks + 7) < 0x7fffffffLL;
  const T* d_o_ = static_cast<const T*>(d_o);
  const T* q_ = static_cast<const T*>(q);
  const T* k_ = static_cast<const T*>(k);
  const T* v_ = static_cast<const T*>(v);
  const T* mask_ = static_cast<const T*>(mask);
  T* dq_ = static_cast<T*>(dq);
  T* dk_ = static_cast<T*>(dk);
  T* dv_ = static_cast<T*>(dv);
  const dim3 grid(static_cast<unsigned>(blocks)), grid_fused(static_cast<unsigned>(2 * ((blocks + 7) / 8 * 8)));
  const dim3 grid_plain(static_cast<unsigned>(blocks * (DP > 128 ? kAttnWideSplit : 1)));
#define MG_LAUNCH(C_, B_)                                                                                            \
  do {                                                                                                               \
    if constexpr (DP <= 64) {                                                                                        \
      if (fused) {                                                                                                   \
        if (!B_ && pipe)                                                                                             \
          hipLaunchKernelGGL((attn_bwd_mfma_kernel<T, DP, C_, B_, !B_>), grid_fused, dim3(kAttnThreads), 0, stream,  \
                             d_o_, q_, k_, v_, mask_, lse, delta.as<float>(), dq_, dk_, dv_, a, scale,               \
                             static_cast<int>(blocks), ps.nlse, ps.ndelta, s_pad);                                   \
        else                                                                                                         \
          hipLaunchKernelGGL((attn_bwd_mfma_kernel<T, DP, C_, B_, false>), grid_fused, dim3(kAttnThreads), 0,        \
                             stream, d_o_, q_, k_, v_, mask_, lse, delta.as<float>(), dq_, dk_, dv_, a, scale,       \
                             static_cast<int>(blocks), ps.nlse, ps.ndelta, s_pad);                                   \
        break;                                                                                                       \
      }                                                                                                              \
      if constexpr (!B_) {                                                                                           \
        if (pipe) {                                                                                                  \
          hipLaunchKernelGGL((attn_dkdv_pipe_kernel<T, DP, C_>), grid, dim3(kAttnThreads), 0, stream, d_o_, q_, k_,  \
                             v_, ps.nlse, ps.ndelta, s_pad, dk_, dv_, a, scale);                                     \
          hipLaunchKernelGGL((attn_dq_pipe_kernel<T, DP, C_>), grid, dim3(kAttnThreads), 0, stream, d_o_, q_, k_,    \
                             v_, lse, delta.as<float>(), dq_, a, scale);                                             \
          break;                                                                                                     \
        }                                                                                                            \
      }                                                                                                              \
    }                                                                                                                \
    hipLaunchKernelGGL((attn_dkdv_mfma_kernel<T, DP, C_, B_>), grid_plain, dim3(kAttnThreads), 0, stream, d_o_, q_,  \
                       k_, v_, mask_, lse, delta.as<float>(), dk_, dv_, a, scale);                                   \
    hipLaunchKernelGGL((attn_dq_mfma_kernel<T, DP, 1, C_, B_>), grid_plain, dim3(kAttnThreads), 0, stream, d_o_, q_, \
                       k_, v_, mask_, lse, delta.as<float>(), dq_, a, scale);                                        \
  } while (0)
  if (causal) MG_LAUNCH(true, false);
  else if (has_bias) MG_LAUNCH(false, true);
  else MG_LAUNCH(false, false);
#undef MG_LAUNCH
  MG_LAUNCH_CHECK();
  return MG_OK;
}

int attn_fwd_mfma(const void* q, const void* k, const void* v, const void* mask, void* o, float* lse, AttnDims a,
                  float scale, bool causal, bool has_bias, int dtype, hipStream_t stream) {
  const bool small = a.D <= 64;
  if (a.D > 128)
    return dtype == MG_BF16 ? fwd_typed<bf16_t, 256>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream)
                            : fwd_typed<f16_t, 256>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream);
  if (dtype == MG_BF16)
    return small ? fwd_typed<bf16_t, 64>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream)
                 : fwd_typed<bf16_t, 128>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream);
  return small ? fwd_typed<f16_t, 64>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream)
               : fwd_typed<f16_t, 128>(q, k, v, mask, o, lse, a, scale, causal, has_bias, stream);
}

int attn_bwd_mfma(const void* d_o, const void* o, const void* q, const void* k, const void* v, const void* mask,
                  const float* lse, void* dq, void* dk, void* dv, AttnDims a, float scale, bool causal, bool has_bias,
                  int dtype, hipStream_t stream) {
  const bool small = a.D <= 64;
  if (a.D > 128)
    return dtype == MG_BF16
               ? bwd_typed<bf16_t, 256>(d_o, o, q, k, v, mask, lse, dq, dk, dv, a, scale, causal, has_bias, stream)
               : bwd_typed<f16_t, 256>(d_o, o, q, k, v, mask, lse, dq, dk, dv, a, scale, causal, has_bias, stream);
  if (dtype == MG_BF16)
    return small ? bwd_typed<bf16_t, 64>(d_o, o, q, k, v, mask, lse, dq, dk, dv, a, scale, causal, has_bias, stream)
                 : bwd_typed<bf16_t, 128>(d_o, o, q, k, v, mask, lse, dq, dk, dv, a, scale, causal, has_bias, stream);
  return small ? bwd_typed<f16_t, 64>(d_o, o, q, k, v, mask, lse, dq, dk, dv, a, scale, causal, has_bias, stream)
               : bwd_typed<f16_t, 128>(d_o, o, q, k, v, mask, lse, dq, dk, dv, a, scale, causal, has_bias, stream);
}

}  // namespace mg
