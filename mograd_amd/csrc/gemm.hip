// C ABI for the matmul family: operand classification, kernel choice, launches.
#include "gemm_impl.h"
#include "mg_deferred.h"
#include "mg_rows.h"

namespace mg {

// A x B with A element (m, k) at a[m * sam + k * sak] and B element (k, n) at
// b[k * sbk + n * sbn]; C row-major (M, N).
struct GemmArgs {
  const void* a;
  const void* b;
  const void* bias;
  void* c;
  int64_t batch, M, N, K;
  int64_t sam, sak, sbk, sbn;
  int64_t bsa, bsb;
  int dtype;
  // Epilogue (see GemmEpilogue): all optional.
  const void* residual = nullptr;
  const void* relu_mask = nullptr;
  int relu = 0;
};

template <typename T>
static GemmEpilogue<T> epilogue_of(const GemmArgs& g) {
  return GemmEpilogue<T>{static_cast<const T*>(g.residual), static_cast<const T*>(g.relu_mask), g.relu};
}

static bool mult4(int64_t v) { return (v & 3) == 0; }

template <bool A_KC, bool B_KC>
static int launch_f32_mfma(const GemmArgs& g, hipStream_t stream) {
  const int tiles_m = static_cast<int>(ceil_div(g.M, kGemmBM));
  const int tiles_n = static_cast<int>(ceil_div(g.N, kGemmBN));
  const int64_t blocks = static_cast<int64_t>(tiles_m) * tiles_n * g.batch;
  if (blocks > 0x7fffffffLL) return fail(MG_ERR_INVALID, "matmul: too many output tiles");
  const int64_t lda = A_KC ? g.sam : g.sak;
  const int64_t ldb = B_KC ? g.sbn : g.sbk;
  const float* a = static_cast<const float*>(g.a);
  const float* b = static_cast<const float*>(g.b);
  const float* bias = static_cast<const float*>(g.bias);
  float* c = static_cast<float*>(g.c);
  // Two workgroups are resident per CU; a larger problem is walked by that many workgroups.
  int64_t grid = 2 * static_cast<int64_t>(device_info().cu_count) * env_int("MOGRAD_HIP_GEMM_F32_ROUNDS", 1);
  if (grid > blocks || env_int("MOGRAD_HIP_GEMM_F32_ROUNDS", 1) == 0) grid = blocks;
  // Tiles copied straight into LDS (gemm_f32_pipe_kernel, same results bit for bit) when K is a
  // multiple of the 32-deep step; MOGRAD_HIP_GEMM_F32_PIPE=0 keeps the register-staged kernel.
  if (g.K % kGemmBK == 0 && env_int("MOGRAD_HIP_GEMM_F32_PIPE", 1) != 0) {
    const int M = static_cast<int>(g.M), N = static_cast<int>(g.N), K = static_cast<int>(g.K);
    const int batches = static_cast<int>(g.batch);
    // An output with fewer tiles than CUs (a 10-class head: 2048 x 10 from K = 4096 is 16
    // tiles) is split along K so that the device is filled; the partial tiles are summed in a
    // fixed order by the same reduction the 16-bit path uses.
    const int64_t cus = device_info().cu_count;
    int splits = 1;
    if (blocks < cus && g.K >= 1024) {
      splits = static_cast<int>(ceil_div(env_int("MOGRAD_HIP_GEMM_SPLITK_WG_PER_CU", 2) * cus, blocks));
      const int max_splits = static_cast<int>(g.K / env_int("MOGRAD_HIP_GEMM_SPLITK_MIN_K", 256));
      if (splits > max_splits) splits = max_splits;
      if (splits > 64) splits = 64;
    }
    if (splits > 1) {
      const int k_per_split = static_cast<int>(ceil_div(ceil_div(g.K, splits), kGemmBK) * kGemmBK);
      splits = static_cast<int>(ceil_div(g.K, k_per_split));
      const int64_t numel = g.batch * g.M * g.N;
      Scratch partial;
      MG_TRY(partial.take(static_cast<int64_t>(splits) * numel * static_cast<int64_t>(sizeof(float))));
      const int64_t work = blocks * splits;
      hipLaunchKernelGGL((gemm_f32_pipe_kernel<A_KC, B_KC, false, true>), dim3(static_cast<unsigned>(work)),
                         dim3(kGemmThreads), 0, stream, a, b, bias, c, partial.as<float>(), M, N, K, lda, ldb, g.N, g.bsa,
                         g.bsb, g.M * g.N, tiles_m, tiles_n, batches, k_per_split, static_cast<int>(work),
                         GemmEpilogue<float>{nullptr, nullptr, 0});
      MG_LAUNCH_CHECK();
      const unsigned rblocks = static_cast<unsigned>(ceil_div(numel, 1024));  // four outputs per thread
      if (bias)
        hipLaunchKernelGGL((gemm_splitk_reduce_kernel<float, true>), dim3(rblocks), dim3(256), 0, stream,
                           partial.as<float>(), bias, c, numel, numel, splits, N, epilogue_of<float>(g));
      else
        hipLaunchKernelGGL((gemm_splitk_reduce_kernel<float, false>), dim3(rblocks), dim3(256), 0, stream,
                           partial.as<float>(), bias, c, numel, numel, splits, N, epilogue_of<float>(g));
      MG_LAUNCH_CHECK();
      return MG_OK;
    }
    float* no_partial = nullptr;
    if (bias)
      hipLaunchKernelGGL((gemm_f32_pipe_kernel<A_KC, B_KC, true, false>), dim3(static_cast<unsigned>(grid)),
                         dim3(kGemmThreads), 0, stream, a, b, bias, c, no_partial, M, N, K, lda, ldb, g.N, g.bsa, g.bsb,
                         g.M * g.N, tiles_m, tiles_n, batches, K, static_cast<int>(blocks), epilogue_of<float>(g));
    else
      hipLaunchKernelGGL((gemm_f32_pipe_kernel<A_KC, B_KC, false, false>), dim3(static_cast<unsigned>(grid)),
                         dim3(kGemmThreads), 0, stream, a, b, bias, c, no_partial, M, N, K, lda, ldb, g.N, g.bsa, g.bsb,
                         g.M * g.N, tiles_m, tiles_n, batches, K, static_cast<int>(blocks), epilogue_of<float>(g));
    MG_LAUNCH_CHECK();
    return MG_OK;
  }
  if (bias)
    hipLaunchKernelGGL((gemm_f32_mfma_kernel<A_KC, B_KC, true>), dim3(static_cast<unsigned>(grid)), dim3(kGemmThreads),
                       0, stream, a, b, bias, c, static_cast<int>(g.M), static_cast<int>(g.N), static_cast<int>(g.K), lda,
                       ldb, g.N, g.bsa, g.bsb, g.M * g.N, tiles_m, tiles_n, static_cast<int>(blocks),
                       epilogue_of<float>(g));
  else
    hipLaunchKernelGGL((gemm_f32_mfma_kernel<A_KC, B_KC, false>), dim3(static_cast<unsigned>(grid)),
                       dim3(kGemmThreads), 0, stream, a, b, bias, c, static_cast<int>(g.M), static_cast<int>(g.N),
                       static_cast<int>(g.K), lda, ldb, g.N, g.bsa, g.bsb, g.M * g.N, tiles_m, tiles_n,
                       static_cast<int>(blocks), epilogue_of<float>(g));
  MG_LAUNCH_CHECK();
  return MG_OK;
}

static bool mult8(int64_t v) { return (v & 7) == 0; }

// gemm_big.hip: the 256 x 256-tile kernel for large 16-bit products (variant 4ksn: k per step,
// copies of the tiles).
int gemm16_big_launch(int dtype, bool a_kc, bool b_kc, int variant, const void* a, const void* b, const void* bias,
                      void* c, int64_t batch, int M, int N, int K, int64_t lda, int64_t ldb, int64_t bsa, int64_t bsb,
                      const void* residual, const void* relu_mask, int relu, hipStream_t stream);

// Into how many K ranges a 16-bit product of `blocks` output tiles is split (1: not at all):
// enough for `wg_per_cu` workgroups per CU, each with at least 256 of K.
static int splitk_16bit_splits(int64_t blocks, int64_t K, int wg_per_cu) {
  const int64_t cus = device_info().cu_count;
  if (blocks >= cus || K < 1024) return 1;
  int splits = static_cast<int>(ceil_div(wg_per_cu * cus, blocks));
  const int max_splits = static_cast<int>(K / env_int("MOGRAD_HIP_GEMM_SPLITK_MIN_K", 256));
  if (splits > max_splits) splits = max_splits;
  if (splits > 64) splits = 64;
  return splits < 1 ? 1 : splits;
}
// The K range of one workgroup, a multiple of the k-step, and the number of ranges that leaves.
static int splitk_16bit_range(int64_t K, int* splits) {
  const int k_per_split = static_cast<int>(ceil_div(ceil_div(K, *splits), kG16BK) * kG16BK);
  *splits = static_cast<int>(ceil_div(K, k_per_split));
  return k_per_split;
}

// 16-bit MFMA path, optionally split along K when the output has too few tiles to fill
// the device (dW of a narrow layer: reduction over thousands of rows into a small matrix).
template <typename T, bool A_KC, bool B_KC, bool RAGGED>
static int launch_16bit_mfma(const GemmArgs& g, hipStream_t stream) {
  const int tiles_m = static_cast<int>(ceil_div(g.M, kGemmBM));
  const int tiles_n = static_cast<int>(ceil_div(g.N, kGemmBN));
  const int64_t tiles = static_cast<int64_t>(tiles_m) * tiles_n;
  const int64_t blocks = tiles * g.batch;
  if (blocks > 0x7fffffffLL) return fail(MG_ERR_INVALID, "matmul: too many output tiles");
  const int64_t lda = A_KC ? g.sam : g.sak;
  const int64_t ldb = B_KC ? g.sbn : g.sbk;
  const T* a = static_cast<const T*>(g.a);
  const T* b = static_cast<const T*>(g.b);
  const T* bias = static_cast<const T*>(g.bias);
  T* c = static_cast<T*>(g.c);
  const int M = static_cast<int>(g.M), N = static_cast<int>(g.N), K = static_cast<int>(g.K);
  const int64_t cus = device_info().cu_count;
  int splits = splitk_16bit_splits(blocks, g.K, env_int("MOGRAD_HIP_GEMM_SPLITK_WG_PER_CU", 2));
  // Tiles copied straight into LDS (gemm_16bit_pipe_kernel) where that measured faster: an
  // operand that is not k-contiguous is transposed by the LDS read instead of in registers
  // (dX 15-25 %, dW 5-20 % faster at Linear-layer shapes, 20-30 % at 4096^3 and up), and long
  // K loops gain from the single barrier per step.  Two k-contiguous operands: from 384 k per
  // workgroup on (2-8 % faster at 16384 rows, 10-25 % at 256-2048 rows), and from 192 for
  // outputs of at most two tiles per CU (8-15 %); shorter K loops, and 192-383 on larger outputs
  // (3-8 % slower there), stay with the register-staged kernel, as does every shape the copy
  // cannot take (MOGRAD_HIP_GEMM16_PIPE_MIN_K moves the 384).  The pair is k per step and copies
  // of the tiles: (32, 2) runs four workgroups per CU, (64, 2) two.
  // MOGRAD_HIP_GEMM16_PIPE = 0 | 322 | 642 | 2322 | 2642 overrides the choice (2xxx: 256 x 128 tiles).
  int pipe = 0;
  if constexpr (!RAGGED) {
    if (g.K % kG16BK == 0 && mult8(g.M) && mult8(g.N)) {
      const int64_t k_wg = ceil_div(g.K, splits);  // the K range one workgroup walks
      if (A_KC && B_KC) {
        const int64_t min_k = env_int("MOGRAD_HIP_GEMM16_PIPE_MIN_K", 384);
        pipe = k_wg >= min_k || (2 * k_wg >= min_k && blocks <= 2 * cus) ? 642 : 0;
      }
      else pipe = k_wg >= 4096 ? 642 : 322;
      // Large products: 256 x 128 tiles (eight waves), a quarter fewer operand bytes per FLOP
      // through L2, once they still give every CU two workgroups (4096^3: 3-11 % faster).
      if (splits <= 1 && g.K >= 1024 && ceil_div(g.M, 256) * tiles_n * g.batch >= 2 * cus) pipe = 2322;
      // Products with a 256 x 256 tile for every CU: four waves of 128 x 128 each, one workgroup
      // per CU (gemm_16bit_big_kernel; 4642: 64 k per step and two copies of the tiles, 4324: 32 k
      // and four; 4096^3 forward 147 -> 121 us, 8192^3 dW 1016 -> 887 us, bit-identical results).
      if (splits <= 1 && g.K >= 1024 && ceil_div(g.M, kGemmBigT) * ceil_div(g.N, kGemmBigT) * g.batch >= cus) pipe = 4642;
      pipe = static_cast<int>(env_int("MOGRAD_HIP_GEMM16_PIPE", pipe));
    }
  }
  if (splits <= 1 && pipe >= 4000) {
    if constexpr (!RAGGED)
      return gemm16_big_launch(g.dtype, A_KC, B_KC, pipe, g.a, g.b, g.bias, g.c, g.batch, M, N, K, lda, ldb, g.bsa, g.bsb,
                               g.residual, g.relu_mask, g.relu, stream);
  }
  if (pipe >= 4000) pipe = 322;
#define MG_GEMM16_LAUNCH(BIAS_, SPLIT_, GRID_, PARTIAL_, KPS_, NSPLIT_, EP_)                                                   \
  do {                                                                                                                 \
    auto launch = [&](auto kernel) {                                                                                   \
      hipLaunchKernelGGL(kernel, GRID_, dim3(kGemmThreads), 0, stream, a, b, bias, c, PARTIAL_, M, N, K, lda, ldb, g.N,  \
                         g.bsa, g.bsb, g.M * g.N, tiles_m, tiles_n, KPS_, NSPLIT_, static_cast<int>(g.batch), EP_);   \
    };                                                                                                                 \
    if constexpr (!RAGGED) {                                                                                           \
      if (pipe == 322) { launch(gemm_16bit_pipe_kernel<T, A_KC, B_KC, BIAS_, SPLIT_, 32, 2>); break; }                 \
      if (pipe == 642) { launch(gemm_16bit_pipe_kernel<T, A_KC, B_KC, BIAS_, SPLIT_, 64, 2>); break; }                 \
    }                                                                                                                  \
    launch(gemm_16bit_mfma_kernel<T, A_KC, B_KC, BIAS_, SPLIT_, RAGGED>);                                              \
  } while (0)
  if (splits <= 1 && (pipe == 2322 || pipe == 2642)) {
    // 256 x 128 tiles, eight waves: a quarter fewer operand bytes per FLOP through L2.
    if constexpr (!RAGGED) {
      const int tiles_m2 = static_cast<int>(ceil_div(g.M, 256));
      const dim3 grid2(static_cast<unsigned>(static_cast<int64_t>(tiles_m2) * tiles_n * g.batch));
      auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid2, dim3(512), 0, stream, a, b, bias, c, static_cast<float*>(nullptr), M, N, K, lda,
                           ldb, g.N, g.bsa, g.bsb, g.M * g.N, tiles_m2, tiles_n, K, 1, static_cast<int>(g.batch),
                           epilogue_of<T>(g));
      };
      if (pipe == 2322) {
        if (bias) launch(gemm_16bit_pipe_kernel<T, A_KC, B_KC, true, false, 32, 2, 256>);
        else launch(gemm_16bit_pipe_kernel<T, A_KC, B_KC, false, false, 32, 2, 256>);
      } else {
        if (bias) launch(gemm_16bit_pipe_kernel<T, A_KC, B_KC, true, false, 64, 2, 256>);
        else launch(gemm_16bit_pipe_kernel<T, A_KC, B_KC, false, false, 64, 2, 256>);
      }
      MG_LAUNCH_CHECK();
      return MG_OK;
    }
  }
  if (pipe > 1000) pipe -= 2000;  // the split-K launch keeps 128 x 128 tiles
  if (splits <= 1) {
    const dim3 grid(static_cast<unsigned>(blocks));
    float* no_partial = nullptr;
    if (bias) MG_GEMM16_LAUNCH(true, false, grid, no_partial, K, 1, epilogue_of<T>(g));
    else MG_GEMM16_LAUNCH(false, false, grid, no_partial, K, 1, epilogue_of<T>(g));
    MG_LAUNCH_CHECK();
    return MG_OK;
  }
  const int k_per_split = splitk_16bit_range(g.K, &splits);
  // Partial tiles: whole 128 x 128 tiles in accumulator order (gemm16_partial_floats); the
  // reduction maps them back onto the contiguous (batch, M, N) output.
  Scratch partial;
  const int64_t slice = gemm16_partial_floats(g.M, g.N, g.batch, 1);
  MG_TRY(partial.take(static_cast<int64_t>(splits) * slice * static_cast<int64_t>(sizeof(float))));
  const int64_t split_grid = gemm_split_grid(tiles, splits, g.batch);
  if (split_grid > 0x7fffffffLL) return fail(MG_ERR_INVALID, "matmul: too many output tiles");
  const dim3 grid(static_cast<unsigned>(split_grid));
  MG_GEMM16_LAUNCH(false, true, grid, partial.as<float>(), k_per_split, splits, (GemmEpilogue<T>{nullptr, nullptr, 0}));
#undef MG_GEMM16_LAUNCH
  MG_LAUNCH_CHECK();
  if (slice / 1024 > 0x7fffffffLL) return fail(MG_ERR_INVALID, "matmul: too many output tiles");
  const unsigned rblocks = static_cast<unsigned>(slice / 1024);  // whole tiles: four outputs per thread
  if (bias)
    hipLaunchKernelGGL((gemm_splitk_reduce_kernel<T, true, true>), dim3(rblocks), dim3(256), 0, stream,
                       partial.as<float>(), bias, c, slice, slice, splits, N, epilogue_of<T>(g), M, tiles_n);
  else
    hipLaunchKernelGGL((gemm_splitk_reduce_kernel<T, false, true>), dim3(rblocks), dim3(256), 0, stream,
                       partial.as<float>(), bias, c, slice, slice, splits, N, epilogue_of<T>(g), M, tiles_n);
  MG_LAUNCH_CHECK();
  return MG_OK;
}

template <typename T>
static int dispatch_16bit(const GemmArgs& g, hipStream_t stream, bool* handled) {
  *handled = false;
  if (g.K <= 0) return MG_OK;
  // Each operand must be contiguous along k or along its other axis.  When leading
  // dimensions, extents and addresses are all multiples of 8 elements the tiles are staged
  // with 16-byte loads; otherwise with element loads (the ragged variant).
  const bool a_kc = g.sak == 1;
  const bool a_mc = g.sam == 1;
  const bool b_kc = g.sbk == 1;
  const bool b_nc = g.sbn == 1;
  const bool worth_it = g.M * g.N >= 64 * 64 || g.K >= 512;
  if (!(worth_it && (a_kc || a_mc) && (b_kc || b_nc))) return MG_OK;
  const bool a_wide = a_kc ? mult8(g.sam) && mult8(g.K) : mult8(g.sak) && mult8(g.M);
  const bool b_wide = b_kc ? mult8(g.sbn) && mult8(g.K) : mult8(g.sbk) && mult8(g.N);
  const bool wide = a_wide && b_wide && aligned16(g.a) && aligned16(g.b) && mult8(g.bsa) && mult8(g.bsb);
  *handled = true;
  if (wide) {
    if (a_kc && b_kc) return launch_16bit_mfma<T, true, true, false>(g, stream);
    if (a_kc) return launch_16bit_mfma<T, true, false, false>(g, stream);
    if (b_kc) return launch_16bit_mfma<T, false, true, false>(g, stream);
    return launch_16bit_mfma<T, false, false, false>(g, stream);
  }
  if (a_kc && b_kc) return launch_16bit_mfma<T, true, true, true>(g, stream);
  if (a_kc) return launch_16bit_mfma<T, true, false, true>(g, stream);
  if (b_kc) return launch_16bit_mfma<T, false, true, true>(g, stream);
  return launch_16bit_mfma<T, false, false, true>(g, stream);
}

template <typename T>
static int launch_generic(const GemmArgs& g, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(ceil_div(g.N, 64)), static_cast<unsigned>(ceil_div(g.M, 64)),
                  static_cast<unsigned>(g.batch));
  if (grid.y > 65535u || grid.z > 65535u) return fail(MG_ERR_INVALID, "matmul: shape exceeds the generic kernel's grid");
  const T* a = static_cast<const T*>(g.a);
  const T* b = static_cast<const T*>(g.b);
  const T* bias = static_cast<const T*>(g.bias);
  T* c = static_cast<T*>(g.c);
  if (bias)
    hipLaunchKernelGGL((gemm_generic_kernel<T, true>), grid, dim3(256), 0, stream, a, b, bias, c, static_cast<int>(g.M),
                       static_cast<int>(g.N), static_cast<int>(g.K), g.sam, g.sak, g.sbk, g.sbn, g.N, g.bsa, g.bsb,
                       g.M * g.N, epilogue_of<T>(g));
  else
    hipLaunchKernelGGL((gemm_generic_kernel<T, false>), grid, dim3(256), 0, stream, a, b, bias, c, static_cast<int>(g.M),
                       static_cast<int>(g.N), static_cast<int>(g.K), g.sam, g.sak, g.sbk, g.sbn, g.N, g.bsa, g.bsb,
                       g.M * g.N, epilogue_of<T>(g));
  MG_LAUNCH_CHECK();
  return MG_OK;
}

int gemm_dispatch(const char* who, const GemmArgs& g_in, hipStream_t stream) {
  const GemmArgs& g = g_in;
  if (!is_float_dtype(g.dtype)) return fail(MG_ERR_INVALID, "%s: unsupported dtype %s", who, dtype_name(g.dtype));
  if (g.batch < 0 || g.M < 0 || g.N < 0 || g.K < 0 || g.M > 0x7fffffffLL || g.N > 0x7fffffffLL || g.K > 0x7fffffffLL)
    return fail(MG_ERR_INVALID, "%s: bad shape batch=%lld M=%lld N=%lld K=%lld", who, static_cast<long long>(g.batch),
                static_cast<long long>(g.M), static_cast<long long>(g.N), static_cast<long long>(g.K));
  if (g.batch == 0 || g.M == 0 || g.N == 0) return MG_OK;
  if (!g.a || !g.b || !g.c) return fail(MG_ERR_INVALID, "%s: null pointer argument", who);

  if (g_in.dtype == MG_F32 && g_in.K > 0) {
    GemmArgs g = g_in;
    // Which dimension of each operand is contiguous, and can it be read 16 bytes at a time?
    bool a_kc = g.sak == 1 && mult4(g.sam) && mult4(g.K) && mult4(g.bsa) && aligned16(g.a);
    const bool a_mc = g.sam == 1 && mult4(g.sak) && mult4(g.M) && mult4(g.bsa) && aligned16(g.a);
    bool b_kc = g.sbk == 1 && mult4(g.sbn) && mult4(g.K) && mult4(g.bsb) && aligned16(g.b);
    const bool b_nc = g.sbn == 1 && mult4(g.sbk) && mult4(g.N) && mult4(g.bsb) && aligned16(g.b);
    // Tiny problems gain nothing from 128x128 tiles.
    const bool worth_it = g.M * g.N >= 64 * 64 || g.K >= env_int("MOGRAD_HIP_GEMM_F32_MIN_K", 128);
    // A thin operand that cannot be read 16 bytes at a time as it lies (the (K, 10) gradient
    // of a 10-class head, read along its 10-wide rows for dW) is first copied k-contiguous:
    // at most one tile of rows, so the copy is a small fraction of the other operand's bytes.
    Scratch a_copy, b_copy;
    const bool deep = g.K >= 512 && mult4(g.K);
    if (deep && !(a_kc || a_mc) && g.M <= kGemmBM && (b_kc || b_nc || g.N <= kGemmBN)) {
      MG_TRY(a_copy.take(g.batch * g.M * g.K * static_cast<int64_t>(sizeof(float))));
      const int64_t shape[3] = {g.batch, g.M, g.K}, strides[3] = {g.bsa, g.sam, g.sak};
      MG_TRY(mg_contiguous(g.a, a_copy.as<float>(), 3, shape, strides, MG_F32, stream));
      g.a = a_copy.as<float>();
      g.sam = g.K, g.sak = 1, g.bsa = g.M * g.K;
      a_kc = true;
    }
    if (deep && !(b_kc || b_nc) && g.N <= kGemmBN && (a_kc || a_mc)) {
      MG_TRY(b_copy.take(g.batch * g.N * g.K * static_cast<int64_t>(sizeof(float))));
      const int64_t shape[3] = {g.batch, g.N, g.K}, strides[3] = {g.bsb, g.sbn, g.sbk};
      MG_TRY(mg_contiguous(g.b, b_copy.as<float>(), 3, shape, strides, MG_F32, stream));
      g.b = b_copy.as<float>();
      g.sbn = g.K, g.sbk = 1, g.bsb = g.N * g.K;
      b_kc = true;
    }
    if (worth_it && (a_kc || a_mc) && (b_kc || b_nc)) {
      if (a_kc && b_kc) return launch_f32_mfma<true, true>(g, stream);
      if (a_kc) return launch_f32_mfma<true, false>(g, stream);
      if (b_kc) return launch_f32_mfma<false, true>(g, stream);
      return launch_f32_mfma<false, false>(g, stream);
    }
  }
  if (g.dtype != MG_F32) {
    bool handled = false;
    const int rc = g.dtype == MG_BF16 ? dispatch_16bit<bf16_t>(g, stream, &handled)
                                      : dispatch_16bit<f16_t>(g, stream, &handled);
    if (handled || rc != MG_OK) return rc;
  }
  switch (g.dtype) {
    case MG_F32: return launch_generic<float>(g, stream);
    case MG_F16: return launch_generic<f16_t>(g, stream);
    default: return launch_generic<bf16_t>(g, stream);
  }
}

int colsum_dispatch(const void* a, void* dst, int64_t outer, int64_t reduce, int64_t inner, int dtype,
                    hipStream_t stream);  // reduce.hip
int ln_bwd(const void* dy, const void* x, const void* gamma, const float* mean, const float* rstd, const void* residual,
           void* dx, void* dgamma, void* dbeta, int64_t rows, int64_t cols, float eps, int dtype,
           mg_stream stream);  // layer_norm.hip

// dX (M,K) = dY (M,N) W (N,K) and dW (N,K) = dY^T X of a 16-bit Linear layer in one launch
// (linear_bwd_16bit_kernel), for the shapes at which launch_16bit_mfma would give both the
// pipelined kernel with 32 k per step and split dW along the rows.  dW comes out bit for bit
// as from its own launch with the same number of K ranges, and so does dX unless its own launch would split it along N (fewer
// dX tiles than CUs): here dX is never split, the dW workgroups fill the device.
// *done = false: not such a shape, nothing launched.
// MOGRAD_HIP_LINEAR_BWD_ONE_LAUNCH=0 switches it off (benchmarks, tests of the equivalence).
// With `ln`, the launch's dX tiles continue as the backward of the LayerNorm whose output X is
// (linear_bwd_ln_16bit_kernel): `dx` then receives that LayerNorm's input gradient (added to
// what it holds when dx_accumulate), dY W itself is not stored, and the LayerNorm's dgamma and
// dbeta follow from one partial row per tile of 128 rows.  Only for the wide tiles of a
// 384-wide input (K == 384); otherwise *done stays false.
struct LinearBwdLayerNorm {
  const void* x;       // the LayerNorm's input (M, K)
  const void* gamma;   // (K)
  const float* mean;   // (M)
  const float* rstd;
  void* dgamma;        // (K)
  void* dbeta;
};

template <typename T>
static int linear_bwd_one_launch(const void* dy, const void* x, const void* w, void* dx, void* dw, int64_t M, int64_t N,
                                 int64_t K, const void* relu_mask, bool dx_accumulate, hipStream_t stream, bool* done,
                                 int64_t dw_rows = -1, void* db = nullptr, bool* db_done = nullptr,
                                 const LinearBwdLayerNorm* ln = nullptr) {
  *done = false;
  if (db_done) *db_done = false;
  if (dw_rows < 0) dw_rows = N;  // rows of dW to write: fewer than N when dY and W came zero-padded
  if (env_int("MOGRAD_HIP_LINEAR_BWD_ONE_LAUNCH", 1) == 0 || env_str("MOGRAD_HIP_GEMM16_PIPE")) return MG_OK;
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL) return MG_OK;
  if (M % kG16BK || N % kG16BK || !mult8(K)) return MG_OK;
  if (!aligned16(dy) || !aligned16(x) || !aligned16(w) || !aligned16(dx) || !aligned16(dw)) return MG_OK;
  if (M * K < 64 * 64 || N * K < 64 * 64) return MG_OK;
  const int64_t cus = device_info().cu_count;
  // Input widths that are multiples of 384 take 128 x 384 output tiles (twelve waves, one
  // workgroup per CU): the three column tiles of a row block share one copy of the dY tile,
  // a third fewer bytes from L2 per FLOP.  MOGRAD_HIP_LINEAR_BWD_WIDE=0: 128 x 128 tiles.
  // Taken when those tiles leave CUs free for dW's K ranges, so that the whole launch is one
  // workgroup per CU, and the layer is wide enough to pay for the larger partial tiles.
  const bool wide = K % kGemmWideBN == 0 && ceil_div(M, kGemmBM) * (K / kGemmWideBN) < cus && N >= 768 &&
                    env_int("MOGRAD_HIP_LINEAR_BWD_WIDE", 1) != 0;
  if (ln && (!wide || K != kGemmWideBN || relu_mask || env_int("MOGRAD_HIP_LINEAR_BWD_STAGES", 2) == 3 ||
             !aligned16(ln->x) || !aligned16(ln->gamma)))
    return MG_OK;
  const int tiles_kk = static_cast<int>(ceil_div(K, wide ? kGemmWideBN : kGemmBN));
  // dW: must be split, each workgroup's rows short enough for the 32-k variant.
  const int w_tiles_m = static_cast<int>(ceil_div(N, kGemmBM));
  const int64_t w_tiles = static_cast<int64_t>(w_tiles_m) * tiles_kk;
  const int x_tiles_m = static_cast<int>(ceil_div(M, kGemmBM));
  const int64_t x_tiles = static_cast<int64_t>(x_tiles_m) * tiles_kk;
  int splits;
  if (wide) {
    // Every workgroup step is the same work (a 128 x 384 x 32 product), so the K ranges of dW
    // are cut to what a CU's share of all steps comes to: with fewer dX tiles than CUs the
    // ranges take the CUs that the tiles leave free, all in one round; otherwise the ranges
    // start first and the tiles fill in behind them.
    const int64_t steps_w = M / kG16BK, steps_x = N / kG16BK;
    const int64_t share = ceil_div(x_tiles * steps_x + w_tiles * steps_w, cus);
    int64_t want = x_tiles < cus ? (cus - x_tiles) / w_tiles : 0;
    if (want < 2) want = ceil_div(steps_w, share);
    const int64_t most = std::min<int64_t>(64, M / 256);
    splits = static_cast<int>(std::max<int64_t>(1, std::min(want, most)));
  } else {
    // One workgroup per CU is enough here: the dX tiles fill the rest of the device, and half
    // the K ranges are half the partial tiles to write and sum (GPT step 3.06 -> 3.00 ms).
    splits = splitk_16bit_splits(w_tiles, M, env_int("MOGRAD_HIP_LINEAR_BWD_SPLIT_WG_PER_CU", 1));
  }
  if (splits <= 1 || ceil_div(M, splits) >= 4096) return MG_OK;
  const int k_per_split = splitk_16bit_range(M, &splits);
  // Every K range of dW and the whole reduction of dX must be whole k-steps (of 32 or 64): the
  // kernels drop a remainder.  Guaranteed by M % kG16BK == 0, N % kG16BK == 0 and ranges cut in
  // units of kG16BK; checked here so that a change to either cannot lose rows silently.
  if (k_per_split % kG16BK != 0 || M % kG16BK != 0 || N % kG16BK != 0) return MG_OK;
  // dX: the 32-k variant.
  if (N >= 4096 || (N >= 1024 && ceil_div(M, 256) * tiles_kk >= 2 * cus)) return MG_OK;
  const int64_t n_dw = gemm_split_grid(w_tiles, splits, 1);
  if (n_dw + x_tiles > 0x7fffffffLL) return MG_OK;

  Scratch partial;
  const int64_t numel = N * K;
  const int64_t slice = gemm16_partial_floats(N, K, 1, 1);  // whole tiles per K range
  MG_TRY(partial.take(static_cast<int64_t>(splits) * slice * static_cast<int64_t>(sizeof(float))));
  const T* dyt = static_cast<const T*>(dy);
  const Gemm16Problem<T> pw{dyt, static_cast<const T*>(x), nullptr, static_cast<T*>(dw), partial.as<float>(),
                            static_cast<int>(N), static_cast<int>(K), static_cast<int>(M),
                            N, K, K, 0, 0, numel, w_tiles_m, tiles_kk, k_per_split, splits, 1,
                            GemmEpilogue<T>{nullptr, nullptr, 0}};
  const Gemm16Problem<T> px{dyt, static_cast<const T*>(w), nullptr, static_cast<T*>(dx), nullptr,
                            static_cast<int>(M), static_cast<int>(K), static_cast<int>(N),
                            N, K, K, 0, 0, M * K, x_tiles_m, tiles_kk, static_cast<int>(N), 1, 1,
                            GemmEpilogue<T>{dx_accumulate ? static_cast<const T*>(dx) : nullptr,
                                            static_cast<const T*>(relu_mask), 0}};
  // The bias gradient rides along: the dW workgroups of the first tile column sum the dY
  // tiles they hold over their K range, and the finishing kernel adds the ranges.  No second
  // pass over dY: (16384, 1536 <- 384) with db 71 -> 60.5 us against dX, dW and a separate
  // mg_sum_axis.  MOGRAD_HIP_LINEAR_BWD_BIAS_IN_LAUNCH=0: the separate column sum.
  Gemm16Problem<T> pw2 = pw;
  // Partial tiles whose sum is deferred are read back at the end of the training step: stored past
  // the caches they do not evict the activations the next kernels read (GPT step 2.48 -> 2.43 ms
  // on one box; MOGRAD_HIP_DEFER_NT_STORE=0 keeps ordinary stores).
  pw2.partial_stream = deferred_current() != nullptr && env_int("MOGRAD_HIP_DEFER_NT_STORE", 1) != 0;
  Scratch db_part;
  int groups = 0;
  if (db && dw_rows == N && env_int("MOGRAD_HIP_LINEAR_BWD_BIAS_IN_LAUNCH", 1) != 0) {
    groups = splits;
    MG_TRY(db_part.take(static_cast<int64_t>(groups) * N * static_cast<int64_t>(sizeof(float))));
    pw2.colsum_part = db_part.as<float>();
  }
  // Three copies of the tiles (two k-steps in flight per workgroup, three workgroups per CU)
  // measured 1 % faster on the GPT step than two copies and four workgroups; four copies no
  // better than two.  MOGRAD_HIP_LINEAR_BWD_STAGES=2 selects two.
  Scratch ln_part_g, ln_part_b;
  if (ln) {
    MG_TRY(ln_part_g.take(static_cast<int64_t>(x_tiles_m) * K * static_cast<int64_t>(sizeof(float))));
    MG_TRY(ln_part_b.take(static_cast<int64_t>(x_tiles_m) * K * static_cast<int64_t>(sizeof(float))));
    Gemm16Problem<T> px2 = px;
    px2.ln = Gemm16LayerNormBwd<T>{static_cast<const T*>(ln->x), static_cast<const T*>(ln->gamma), ln->mean, ln->rstd,
                                   ln_part_g.as<float>(), ln_part_b.as<float>()};
    hipLaunchKernelGGL((linear_bwd_ln_16bit_kernel<T>), dim3(static_cast<unsigned>(n_dw + x_tiles)), dim3(2 * kGemmWideBN),
                       0, stream, pw2, px2, static_cast<int>(n_dw));
  } else if (wide && env_int("MOGRAD_HIP_LINEAR_BWD_STAGES", 2) == 3)  // 32 k per step, three copies: 3-4 % slower
    hipLaunchKernelGGL((linear_bwd_16bit_kernel<T, 3, kGemmWideBN>), dim3(static_cast<unsigned>(n_dw + x_tiles)),
                       dim3(2 * kGemmWideBN), 0, stream, pw2, px, static_cast<int>(n_dw));
  else if (wide)  // 64 k per step, two copies (128 KB of LDS): half the barriers, whole cache lines of dY
    hipLaunchKernelGGL((linear_bwd_16bit_kernel<T, 2, kGemmWideBN, 64>), dim3(static_cast<unsigned>(n_dw + x_tiles)),
                       dim3(2 * kGemmWideBN), 0, stream, pw2, px, static_cast<int>(n_dw));
  else if (env_int("MOGRAD_HIP_LINEAR_BWD_STAGES", 3) == 2)
    hipLaunchKernelGGL((linear_bwd_16bit_kernel<T, 2>), dim3(static_cast<unsigned>(n_dw + x_tiles)), dim3(kGemmThreads), 0,
                       stream, pw2, px, static_cast<int>(n_dw));
  else
    hipLaunchKernelGGL((linear_bwd_16bit_kernel<T, 3>), dim3(static_cast<unsigned>(n_dw + x_tiles)), dim3(kGemmThreads), 0,
                       stream, pw2, px, static_cast<int>(n_dw));
  MG_LAUNCH_CHECK();
  if (ln) {  // the tiles' partial rows of dgamma / dbeta: summed now, or left on the deferred list
    reduce_partials_or_defer<T>(ln_part_g, static_cast<T*>(ln->dgamma), &ln_part_b, static_cast<T*>(ln->dbeta), x_tiles_m,
                                K, static_cast<int>(cus), stream);
    MG_LAUNCH_CHECK();
  }
  const int dw_blocks = static_cast<int>(slice / 1024);  // 256 threads, four consecutive partial values each
  const int db_blocks = groups > 0 ? static_cast<int>(ceil_div(N, 64)) : 0;
  if (DeferredList* dl = deferred_current()) {
    // The sums of the K ranges are left to mg_finish_deferred (same code, same order).
    dl->push(kDeferSplitK, partial.as<float>(), dw, slice, static_cast<int>(dw_rows), static_cast<int>(K), splits,
             ceil_div(slice / 4, 1024));
    dl->hold(partial);
    if (groups > 0) {
      dl->push(kDeferBiasRows, db_part.as<float>(), db, 0, 0, static_cast<int>(N), groups, ceil_div(db_blocks, 4));
      dl->hold(db_part);
    }
    if (db_done) *db_done = groups > 0;
    *done = true;
    return MG_OK;
  }
  hipLaunchKernelGGL((linear_bwd_finish_kernel<T>), dim3(static_cast<unsigned>(dw_blocks + db_blocks)), dim3(256), 0,
                     stream, partial.as<float>(), static_cast<T*>(dw), static_cast<int>(dw_rows), slice, splits,
                     static_cast<int>(K), dw_blocks, db_part.as<float>(), static_cast<T*>(db), groups,
                     static_cast<int>(N));
  MG_LAUNCH_CHECK();
  if (db_done) *db_done = groups > 0;
  *done = true;
  return MG_OK;
}

// dst (rows, cols_to) = src (rows, cols) with zero columns appended; cols_to is a multiple of 8
// and dst 16-byte aligned.  One thread per 8 output columns.
template <typename T>
__global__ __launch_bounds__(256) void pad_columns_kernel(const T* __restrict__ src, T* __restrict__ dst, int64_t rows,
                                                          int cols, int cols_to) {
  const int chunks = cols_to / 8;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= rows * chunks) return;
  const int64_t r = i / chunks;
  const int c0 = static_cast<int>(i % chunks) * 8;
  T v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = c0 + e < cols ? src[r * cols + c0 + e] : from_float<T>(0.f);
  *reinterpret_cast<uint4*>(dst + r * cols_to + c0) = *reinterpret_cast<const uint4*>(v);
}

// A layer whose width N is not a multiple of the k-step (a 65-symbol vocabulary) cannot take
// the pipelined kernels as it lies: rows of dY start at odd addresses, and both products
// would go to the element-staged kernel (3-4 % of the matrix cores busy).  Here dY gets
// zero columns and W zero rows up to the next multiple of 64 (copies of M x N and N x K
// elements, small beside X and dX), the padded layer goes through the common launch, and
// only the first N rows of dW are written.  The padding adds exact zeros to every sum.
template <typename T>
static int linear_bwd_padded(const void* dy, const void* x, const void* w, void* dx, void* dw, int64_t M, int64_t N,
                             int64_t K, const void* relu_mask, bool dx_accumulate, hipStream_t stream, bool* done) {
  *done = false;
  const int64_t n_to = ceil_div(N, kG16BK) * kG16BK;
  if (N % kG16BK == 0 || n_to > 2 * N || M % kG16BK || !mult8(K) || M < 1024 || n_to * K > 0x7fffffffLL) return MG_OK;
  if (env_int("MOGRAD_HIP_LINEAR_BWD_ONE_LAUNCH", 1) == 0 || env_str("MOGRAD_HIP_GEMM16_PIPE")) return MG_OK;
  Scratch dy_pad, w_pad;
  MG_TRY(dy_pad.take(M * n_to * static_cast<int64_t>(sizeof(T))));
  MG_TRY(w_pad.take(n_to * K * static_cast<int64_t>(sizeof(T))));
  // W: rows appended to a row-major array, i.e. one row of N * K elements padded to n_to * K
  const int64_t w_chunks = n_to * K / 8, dy_chunks = M * (n_to / 8);
  hipLaunchKernelGGL((pad_columns_kernel<T>), dim3(static_cast<unsigned>(ceil_div(w_chunks, 256))), dim3(256), 0, stream,
                     static_cast<const T*>(w), w_pad.as<T>(), static_cast<int64_t>(1), static_cast<int>(N * K),
                     static_cast<int>(n_to * K));
  MG_LAUNCH_CHECK();
  hipLaunchKernelGGL((pad_columns_kernel<T>), dim3(static_cast<unsigned>(ceil_div(dy_chunks, 256))), dim3(256), 0, stream,
                     static_cast<const T*>(dy), dy_pad.as<T>(), M, static_cast<int>(N), static_cast<int>(n_to));
  MG_LAUNCH_CHECK();
  return linear_bwd_one_launch<T>(dy_pad.as<T>(), x, w_pad.as<T>(), dx, dw, M, n_to, K, relu_mask, dx_accumulate, stream,
                                  done, N);
}

// *done: dX and dW are on their way; *db_done: so is db (else the caller sums dY's columns).
int linear_bwd_products(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db, int64_t M, int64_t N,
                        int64_t K, const void* relu_mask, bool dx_accumulate, int dtype, hipStream_t stream, bool* done,
                        bool* db_done, const LinearBwdLayerNorm* ln = nullptr) {
  *done = false;
  *db_done = false;
  if (ln) {  // only the one launch has the LayerNorm continuation
    if (dtype == MG_BF16)
      return linear_bwd_one_launch<bf16_t>(dy, x, w, dx, dw, M, N, K, relu_mask, dx_accumulate, stream, done, -1, db,
                                           db_done, ln);
    if (dtype == MG_F16)
      return linear_bwd_one_launch<f16_t>(dy, x, w, dx, dw, M, N, K, relu_mask, dx_accumulate, stream, done, -1, db,
                                          db_done, ln);
    return MG_OK;
  }
  if (dtype == MG_BF16) {
    MG_TRY(linear_bwd_one_launch<bf16_t>(dy, x, w, dx, dw, M, N, K, relu_mask, dx_accumulate, stream, done, -1, db,
                                         db_done));
    if (!*done) MG_TRY(linear_bwd_padded<bf16_t>(dy, x, w, dx, dw, M, N, K, relu_mask, dx_accumulate, stream, done));
  } else if (dtype == MG_F16) {
    MG_TRY(linear_bwd_one_launch<f16_t>(dy, x, w, dx, dw, M, N, K, relu_mask, dx_accumulate, stream, done, -1, db,
                                        db_done));
    if (!*done) MG_TRY(linear_bwd_padded<f16_t>(dy, x, w, dx, dw, M, N, K, relu_mask, dx_accumulate, stream, done));
  }
  return MG_OK;
}

}  // namespace mg

extern "C" {

int mg_matmul(const void* a, const void* b, void* dst, int64_t batch, int64_t M, int64_t N, int64_t K, int64_t lda0,
              int64_t lda1, int64_t ldb0, int64_t ldb1, int64_t batch_stride_a, int64_t batch_stride_b, int dtype,
              mg_stream stream) {
  mg::GemmArgs g{a, b, nullptr, dst, batch, M, N, K, lda0, lda1, ldb0, ldb1, batch_stride_a, batch_stride_b, dtype};
  return mg::gemm_dispatch("matmul", g, mg::to_stream(stream));
}

int mg_matmul_bt(const void* a, const void* b, void* dst, int64_t batch, int64_t M, int64_t N, int64_t K, int64_t lda0,
                 int64_t lda1, int64_t ldb0, int64_t ldb1, int64_t batch_stride_a, int64_t batch_stride_b, int dtype,
                 mg_stream stream) {
  // B arrives as (N, K): element (k, n) of the product's right operand is b[n * ldb0 + k * ldb1].
  mg::GemmArgs g{a, b, nullptr, dst, batch, M, N, K, lda0, lda1, ldb1, ldb0, batch_stride_a, batch_stride_b, dtype};
  return mg::gemm_dispatch("matmul", g, mg::to_stream(stream));
}

int mg_matmul_bias_bt(const void* a, const void* b, const void* bias, void* dst, int64_t batch, int64_t M, int64_t N,
                      int64_t K, int64_t lda0, int64_t lda1, int64_t ldb0, int64_t ldb1, int64_t batch_stride_a,
                      int64_t batch_stride_b, int dtype, mg_stream stream) {
  if (!bias) return mg::fail(MG_ERR_INVALID, "matmul_bias: null bias pointer");
  mg::GemmArgs g{a, b, bias, dst, batch, M, N, K, lda0, lda1, ldb1, ldb0, batch_stride_a, batch_stride_b, dtype};
  return mg::gemm_dispatch("matmul_bias", g, mg::to_stream(stream));
}

int mg_matmul_bt_add(const void* a, const void* b, const void* residual, void* dst, int64_t batch, int64_t M, int64_t N,
                     int64_t K, int64_t lda0, int64_t lda1, int64_t ldb0, int64_t ldb1, int64_t batch_stride_a,
                     int64_t batch_stride_b, int dtype, mg_stream stream) {
  if (!residual) return mg::fail(MG_ERR_INVALID, "matmul_add: null residual pointer");
  mg::GemmArgs g{a, b, nullptr, dst, batch, M, N, K, lda0, lda1, ldb1, ldb0, batch_stride_a, batch_stride_b, dtype};
  g.residual = residual;
  return mg::gemm_dispatch("matmul_add", g, mg::to_stream(stream));
}

int mg_matmul_bias_relu_bt(const void* a, const void* b, const void* bias, void* dst, int64_t batch, int64_t M, int64_t N,
                           int64_t K, int64_t lda0, int64_t lda1, int64_t ldb0, int64_t ldb1, int64_t batch_stride_a,
                           int64_t batch_stride_b, int dtype, mg_stream stream) {
  if (!bias) return mg::fail(MG_ERR_INVALID, "matmul_bias_relu: null bias pointer");
  mg::GemmArgs g{a, b, bias, dst, batch, M, N, K, lda0, lda1, ldb1, ldb0, batch_stride_a, batch_stride_b, dtype};
  g.relu = 1;
  return mg::gemm_dispatch("matmul_bias_relu", g, mg::to_stream(stream));
}

static int linear_bwd_impl(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db, int64_t M,
                           int64_t N, int64_t K, bool dx_accumulate, bool x_is_relu_output, int dtype, mg_stream stream) {
  hipStream_t s = mg::to_stream(stream);
  if (x_is_relu_output && dx && !x) return mg::fail(MG_ERR_INVALID, "linear_bwd: x is needed as the relu mask");
  if (dx && dw && dy && x && w) {
    bool done = false, db_done = false;
    MG_TRY(mg::linear_bwd_products(dy, x, w, dx, dw, db, M, N, K, x_is_relu_output ? x : nullptr, dx_accumulate, dtype,
                                   s, &done, &db_done));
    if (done) {
      if (db && !db_done) MG_TRY(mg::colsum_dispatch(dy, db, 1, M, N, dtype, s));
      return MG_OK;
    }
  }
  if (dx) {  // dX (M,K) = dY (M,N) x W (N,K): reduction over N, W read as an n-contiguous right operand
    mg::GemmArgs g{dy, w, nullptr, dx, 1, M, K, N, N, 1, K, 1, 0, 0, dtype};
    if (x_is_relu_output) {
      if (!x) return mg::fail(MG_ERR_INVALID, "linear_bwd: x is needed as the relu mask");
      g.relu_mask = x;  // (M, K), laid out like dX
    }
    if (dx_accumulate) g.residual = dx;
    MG_TRY(mg::gemm_dispatch("linear_bwd(dx)", g, s));
  }
  if (dw) {  // dW (N,K) = dY^T (N,M) x X (M,K): reduction over M, dY read as an m-contiguous left operand
    mg::GemmArgs g{dy, x, nullptr, dw, 1, N, K, M, 1, N, K, 1, 0, 0, dtype};
    MG_TRY(mg::gemm_dispatch("linear_bwd(dw)", g, s));
  }
  if (db) MG_TRY(mg::colsum_dispatch(dy, db, 1, M, N, dtype, s));
  return MG_OK;
}

int mg_linear_bwd(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db, int64_t M, int64_t N,
                  int64_t K, int dtype, mg_stream stream) {
  return linear_bwd_impl(dy, x, w, dx, dw, db, M, N, K, false, false, dtype, stream);
}

int mg_linear_bwd_fused(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db, int64_t M, int64_t N,
                        int64_t K, int dx_accumulate, int x_is_relu_output, int dtype, mg_stream stream) {
  return linear_bwd_impl(dy, x, w, dx, dw, db, M, N, K, dx_accumulate != 0, x_is_relu_output != 0, dtype, stream);
}

int mg_linear_bwd_deferred(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db, int64_t M,
                           int64_t N, int64_t K, int dx_accumulate, int x_is_relu_output, int dtype, int grad_dtype,
                           mg_deferred list, mg_stream stream) {
  if (!mg::is_float_dtype(dtype))
    return mg::fail(MG_ERR_INVALID, "linear_bwd_deferred: unsupported dtype %s", mg::dtype_name(dtype));
  MG_TRY(mg::deferred_check("linear_bwd_deferred", list, dtype, grad_dtype));
  if (M < 0 || N < 0 || K < 0) return mg::fail(MG_ERR_INVALID, "linear_bwd_deferred: negative size");
  mg::DeferredScope scope(static_cast<mg::DeferredList*>(list), dtype, grad_dtype);
  void *dw_use, *db_use;
  MG_TRY(scope.substitute(dw, N * K, &dw_use));
  MG_TRY(scope.substitute(db, N, &db_use));
  MG_TRY(linear_bwd_impl(dy, x, w, dx, dw_use, db_use, M, N, K, dx_accumulate != 0, x_is_relu_output != 0, dtype, stream));
  return scope.finish(mg::to_stream(stream));
}

int mg_linear_bwd_layer_norm_bwd(const void* dy, const void* x, const void* w, const void* ln_x, const void* gamma,
                                 const float* mean, const float* rstd, void* dx, void* dw, void* db, void* dgamma,
                                 void* dbeta, int64_t M, int64_t N, int64_t K, int dx_accumulate, int dtype,
                                 int grad_dtype, mg_deferred list, mg_stream stream) {
  const char* who = "linear_bwd_layer_norm_bwd";
  if (!mg::is_float_dtype(dtype)) return mg::fail(MG_ERR_INVALID, "%s: unsupported dtype %s", who, mg::dtype_name(dtype));
  if (M < 0 || N < 0 || K <= 0) return mg::fail(MG_ERR_INVALID, "%s: bad size", who);
  if (!dy || !x || !w || !ln_x || !gamma || !mean || !rstd || !dx || !dw || !dgamma || !dbeta)
    return mg::fail(MG_ERR_INVALID, "%s: null pointer argument", who);
  if (list) MG_TRY(mg::deferred_check(who, list, dtype, grad_dtype));
  else if (grad_dtype != dtype) return mg::fail(MG_ERR_INVALID, "%s: without a deferred list the gradients have the tensors' dtype", who);
  hipStream_t s = mg::to_stream(stream);
  auto run = [&](void* dw_use, void* db_use, void* dg_use, void* dbt_use) -> int {
    bool done = false, db_done = false;
    const mg::LinearBwdLayerNorm ln{ln_x, gamma, mean, rstd, dg_use, dbt_use};
    MG_TRY(mg::linear_bwd_products(dy, x, w, dx, dw_use, db_use, M, N, K, nullptr, dx_accumulate != 0, dtype, s, &done,
                                   &db_done, &ln));
    if (done) {
      if (db_use && !db_done) MG_TRY(mg::colsum_dispatch(dy, db_use, 1, M, N, dtype, s));
      return MG_OK;
    }
    // Other shapes: dY W into a scratch tensor with the separate entry's kernels, then the LayerNorm backward.
    mg::Scratch dy_ln;
    MG_TRY(dy_ln.take(M * K * static_cast<int64_t>(mg::dtype_size(dtype))));
    MG_TRY(linear_bwd_impl(dy, x, w, dy_ln.as<char>(), dw_use, db_use, M, N, K, false, false, dtype, stream));
    return mg::ln_bwd(dy_ln.as<char>(), ln_x, gamma, mean, rstd, dx_accumulate ? dx : nullptr, dx, dg_use, dbt_use, M, K,
                      0.f, dtype, stream);
  };
  if (!list) return run(dw, db, dgamma, dbeta);
  mg::DeferredScope scope(static_cast<mg::DeferredList*>(list), dtype, grad_dtype);
  void *dw_use, *db_use, *dg_use, *dbt_use;
  MG_TRY(scope.substitute(dw, N * K, &dw_use));
  MG_TRY(scope.substitute(db, N, &db_use));
  MG_TRY(scope.substitute(dgamma, K, &dg_use));
  MG_TRY(scope.substitute(dbeta, K, &dbt_use));
  MG_TRY(run(dw_use, db_use, dg_use, dbt_use));
  return scope.finish(s);
}

}  // extern "C"
