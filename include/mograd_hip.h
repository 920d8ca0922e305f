/*
 * mograd_hip.h — C ABI of libmograd_hip.so: MI355X (gfx950) kernels for the backward hot
 * path of mograd (LayerNorm, softmax cross-entropy, Linear gradients, flash attention),
 * plus the stream and caching-pool plumbing those kernels need.
 *
 * Conventions
 *   - Every function returns 0 on success and a non-zero mg_status on failure;
 *     mg_last_error() then returns a thread-local message.  The reference raises Mojo
 *     errors in the same situations; a binding re-raises from the message.
 *   - All data pointers are DEVICE pointers unless a parameter is documented as host.
 *   - The caller owns inputs and outputs.  Outputs need no initialisation.  Scratch is
 *     taken from the library's pool and returned before the call returns; this is safe
 *     because all work of one call is enqueued on the one stream passed in, and the pool
 *     hands memory back out only to later calls (the reference's single in-order-stream
 *     contract, mograd/memory.mojo:27-31).  This makes the library a one-stream-per-device
 *     library: every entry point that takes scratch (the LayerNorm, cross-entropy, Linear
 *     and attention backward entries, split products, mg_sum_axis, mg_scatter_add and the
 *     `_deferred` forms) returns its blocks to the pool while its kernels are still queued,
 *     untagged by stream, so calls issued on two streams of one device that overlap in
 *     time may be handed the same block.  Use one stream per device, or order the streams
 *     with events so that such calls never overlap.
 *   - `stream` is a hipStream_t passed as void*; NULL is the default stream.  No function
 *     synchronises the host unless its comment says so.
 *   - The symbols are new names: the reference's own `mograd_*` exports use the Mojo ABI
 *     with Mojo-only argument types (mograd/runtime/gpu/kernels/dispatch.mojo:83-554)
 *     and cannot be honoured from C.  Each declaration cites the export it replaces.
 */
#ifndef MOGRAD_HIP_H
#define MOGRAD_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types.  The reference supports f16, f32 and i64 (mograd/buffer.mojo:136);
 * bf16 and i32 are additions. */
typedef enum mg_dtype {
  MG_F32 = 0,
  MG_F16 = 1,
  MG_BF16 = 2,
  MG_I32 = 3,
  MG_I64 = 4
} mg_dtype;

typedef enum mg_status {
  MG_OK = 0,
  MG_ERR_INVALID = 1,     /* bad argument (shape, dtype, alignment, flag combination) */
  MG_ERR_UNSUPPORTED = 2, /* valid request this build has no kernel for */
  MG_ERR_HIP = 3,         /* a HIP runtime call failed; message carries hipGetErrorString */
  MG_ERR_OOM = 4          /* device allocation failed after flushing the cache */
} mg_status;

typedef void* mg_stream;

/* ------------------------------------------------------------------------------------ */
/* Library, errors, streams                                                              */
/* ------------------------------------------------------------------------------------ */

/* Version string "mograd_hip x.y (gfx950)". */
const char* mg_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char* mg_last_error(void);

/* Selects `device` for this thread and reads its properties (CU count).  Optional:
 * every entry point initialises lazily on the current device.
 * Replaces Device() construction, mograd/device_ctx.mojo:44-54. */
int mg_init(int device);

/* Number of compute units of the current device (the reference's MULTIPROCESSOR_COUNT,
 * kernels/normalization.mojo:322). */
int mg_device_cu_count(void);

/* One in-order stream, default priority.  Replaces the DeviceContext's stream. */
int mg_stream_create(mg_stream* out);
int mg_stream_destroy(mg_stream stream);
/* Blocks the host until `stream` drains (ctx.synchronize(), scheduler.mojo:80). */
int mg_stream_sync(mg_stream stream);

/* Events on a stream, for timing kernels where they run.  mg_event_elapsed_ms blocks the
 * host until `stop` has completed.  (The reference times with perf_counter_ns around a
 * synchronize, mograd/debug.mojo:98-114.) */
typedef void* mg_event;
int mg_event_create(mg_event* out);
int mg_event_destroy(mg_event event);
int mg_event_record(mg_event event, mg_stream stream);
int mg_event_elapsed_ms(mg_event start, mg_event stop, float* ms);

/* Host <-> device copies and fills for buffers the caller owns.  The copies are
 * synchronous with respect to the host (they return when the bytes have arrived).
 * Replace Buffer.from_data / to_list / full, mograd/buffer.mojo. */
int mg_copy_to_device(void* dst, const void* host_src, int64_t nbytes, mg_stream stream);
int mg_copy_to_host(void* host_dst, const void* src, int64_t nbytes, mg_stream stream);
int mg_copy_device(void* dst, const void* src, int64_t nbytes, mg_stream stream);
/* dst[i] = value for i < numel, converted to `dtype` (any mg_dtype).  Asynchronous. */
int mg_fill(void* dst, double value, int64_t numel, int dtype, mg_stream stream);

/* ------------------------------------------------------------------------------------ */
/* Caching device-memory pool (mograd/memory.mojo)                                       */
/* ------------------------------------------------------------------------------------ */

typedef struct mg_pool_stats {
  int64_t allocated_bytes; /* class bytes handed out and not yet returned */
  int64_t reserved_bytes;  /* allocated + cached in free lists */
  int64_t peak_allocated;
  int64_t peak_reserved;
  int64_t alloc_count; /* real hipMalloc calls */
  int64_t hit_count;
  int64_t miss_count;
  int64_t free_count; /* returns to the free lists */
} mg_pool_stats;

/* Size class of a request: multiples of prev_pow2(n)/8, minimum 512 B.
 * memory.mojo:59-72 (round_class). */
int64_t mg_round_class(int64_t nbytes);

/* 1 unless the environment has MOGRAD_POOL=0 (memory.mojo:132). */
int mg_pool_enabled(void);

/* Returns storage of at least nbytes, reusing a cached block of the same class.  On
 * hipMalloc failure the cache is emptied, the device synchronised and the allocation
 * retried once (memory.mojo:242-295, take_storage/_driver_alloc). */
int mg_pool_alloc(void** out, int64_t nbytes);

/* Returns a block to its class free list (Storage.__deinit__/_release,
 * memory.mojo:227-311).  Memory goes back to the driver only in mg_pool_empty_cache. */
int mg_pool_free(void* ptr);

/* Frees every cached block to the driver; reserved == allocated afterwards
 * (memory.mojo:353-362). */
int mg_pool_empty_cache(void);

/* memory_stats, memory.mojo:377-382. */
int mg_pool_get_stats(mg_pool_stats* out);

/* memory_summary, memory.mojo:385-412.  Writes at most cap-1 bytes plus NUL into the
 * HOST buffer `buf`; returns the full length needed. */
int64_t mg_pool_summary(char* buf, int64_t cap);

/* ------------------------------------------------------------------------------------ */
/* LayerNorm over the last axis.  rows = numel / cols, cols = last dim                   */
/* (kernels/dispatch.mojo:295-313,336-357).  dtype in {F32, F16, BF16}; math in fp32.     */
/* ------------------------------------------------------------------------------------ */

/* y = (x - mean) * rstd * gamma + beta, biased variance.
 * Replaces mograd_layer_norm_fwd, kernels/__init__.mojo:1309-1334. */
int mg_layer_norm_fwd(const void* x, const void* gamma, const void* beta, void* y, int64_t rows,
                      int64_t cols, float eps, int dtype, mg_stream stream);

/* Same, and also writes the per-row statistics (fp32, `rows` each) for the backward to
 * reuse.  No counterpart in the reference, whose forward has one output
 * (mograd/runtime/__init__.mojo:425-426). */
int mg_layer_norm_fwd_stats(const void* x, const void* gamma, const void* beta, void* y,
                            float* mean, float* rstd, int64_t rows, int64_t cols, float eps,
                            int dtype, mg_stream stream);

/* dx (rows, cols), dgamma (cols), dbeta (cols) from dy, x, gamma.  dgamma/dbeta are
 * fully overwritten (the reference's caller zero-fills them first; not needed here).
 * Two launches: row kernel with per-group partial sums, then a column reduction; no
 * atomics.  Replaces mograd_layer_norm_bwd, kernels/__init__.mojo:1337-1366
 * (kernels/normalization.mojo:85-400). */
int mg_layer_norm_bwd(const void* dy, const void* x, const void* gamma, void* dx, void* dgamma,
                      void* dbeta, int64_t rows, int64_t cols, float eps, int dtype,
                      mg_stream stream);

/* Same with the forward's saved statistics instead of recomputing them from x. */
int mg_layer_norm_bwd_stats(const void* dy, const void* x, const void* gamma, const float* mean,
                            const float* rstd, void* dx, void* dgamma, void* dbeta, int64_t rows,
                            int64_t cols, int dtype, mg_stream stream);

/* mg_layer_norm_bwd_stats with the result added to `residual` (same shape and dtype as dx;
 * may be dx itself: in-place accumulation into a gradient that already holds the skip
 * connection's share).  dx = round(gradient) + residual, bit for bit what
 * mg_layer_norm_bwd_stats followed by mg_add gives.  The reference has no such form: its
 * graph accumulates gradients with a separate ADD node (Grad.accum, mograd/grad.mojo:93-95). */
int mg_layer_norm_bwd_stats_add(const void* dy, const void* x, const void* gamma, const float* mean,
                                const float* rstd, const void* residual, void* dx, void* dgamma,
                                void* dbeta, int64_t rows, int64_t cols, int dtype, mg_stream stream);

/* ------------------------------------------------------------------------------------ */
/* Softmax cross-entropy.  N = numel / C rows, C = last dim                              */
/* (kernels/__init__.mojo:1386-1387).  dtype in {F32, F16, BF16}; math in fp32.           */
/* ------------------------------------------------------------------------------------ */

/* loss[0] = -(1/N) sum_rows sum_c labels * log_softmax(logits), DENSE labels of the
 * logits' shape and dtype (one-hot or soft).  Unlike the reference this does not
 * synchronise the host.  Replaces mograd_cross_entropy, kernels/__init__.mojo:1374-1408
 * (kernels/cross_entropy.mojo:14-77,155-177). */
int mg_cross_entropy(const void* logits, const void* labels, void* loss, int64_t N, int64_t C,
                     int dtype, mg_stream stream);

/* dlogits = (softmax(logits) - labels) * upstream[0] / N.  `upstream` is a 1-element
 * device buffer of `dtype`.  Replaces mograd_cross_entropy_grad,
 * kernels/__init__.mojo:1462-1489 (kernels/cross_entropy.mojo:185-241). */
int mg_cross_entropy_grad(const void* logits, const void* labels, const void* upstream,
                          void* dlogits, int64_t N, int64_t C, int dtype, mg_stream stream);

/* Strided forms: logits and labels are `rank`-dimensional views sharing `shape` (HOST
 * array) with independent element strides (HOST arrays); the last dim is C.  The output
 * of the gradient is contiguous.  Replace mograd_cross_entropy_strided and
 * mograd_cross_entropy_grad_strided, kernels/__init__.mojo:1411-1454,1492-1528. */
int mg_cross_entropy_strided(const void* logits, const void* labels, void* loss, int rank,
                             const int64_t* shape, const int64_t* logits_strides,
                             const int64_t* labels_strides, int dtype, mg_stream stream);
int mg_cross_entropy_grad_strided(const void* logits, const void* labels, const void* upstream,
                                  void* dlogits, int rank, const int64_t* shape,
                                  const int64_t* logits_strides, const int64_t* labels_strides,
                                  int dtype, mg_stream stream);

/* Integer class ids instead of dense labels: `ids` holds N values of `id_dtype`
 * (MG_I32 or MG_I64), each in [0, C).  Results equal the dense forms with
 * labels = one_hot(ids).  No counterpart in the reference (labels reach it as
 * one_hot(...).cast(f32), examples/mnist/train.mojo:36).
 *   _ids        loss only        (reads logits once)
 *   _grad_ids   dlogits only     (reads logits once, writes dlogits once)
 *   _fused_ids  loss and dlogits in one pass over the logits.
 * `upstream` may be NULL, meaning 1. */
int mg_cross_entropy_ids(const void* logits, const void* ids, void* loss, int64_t N, int64_t C,
                         int dtype, int id_dtype, mg_stream stream);
int mg_cross_entropy_grad_ids(const void* logits, const void* ids, const void* upstream,
                              void* dlogits, int64_t N, int64_t C, int dtype, int id_dtype,
                              mg_stream stream);
int mg_cross_entropy_fused_ids(const void* logits, const void* ids, const void* upstream,
                               void* loss, void* dlogits, int64_t N, int64_t C, int dtype,
                               int id_dtype, mg_stream stream);
/* mg_cross_entropy_fused_ids for callers that cannot allocate (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same arguments, kernels
 * and results, but the per-row loss terms go to a static device array of
 * MG_CE_NOALLOC_MAX_ROWS floats (4 MiB per GPU, held until the process ends) instead of a
 * pool block, and the call makes no hipMalloc/hipFree and takes nothing from the pool.
 * N above MG_CE_NOALLOC_MAX_ROWS is rejected with MG_ERR_INVALID.  Every call on a GPU
 * shares that GPU's array: calls that overlap on one GPU (different streams) race; calls
 * on one stream are ordered.  The array's device address is looked up once per device
 * (in mg_init, else on the first call there), so call mg_init or make one call before
 * starting a capture.  No counterpart in the reference. */
#define MG_CE_NOALLOC_MAX_ROWS (1 << 20)
int mg_cross_entropy_fused_ids_noalloc(const void* logits, const void* ids, const void* upstream,
                                       void* loss, void* dlogits, int64_t N, int64_t C, int dtype,
                                       int id_dtype, mg_stream stream);

/* Dense-label loss and dlogits in one pass. */
int mg_cross_entropy_fused(const void* logits, const void* labels, const void* upstream,
                           void* loss, void* dlogits, int64_t N, int64_t C, int dtype,
                           mg_stream stream);

/* ------------------------------------------------------------------------------------ */
/* Matmul family.  dst is always contiguous (batch, M, N).                               */
/* Operand strides are in elements.  dtype in {F32, F16, BF16}; fp32 accumulation.        */
/* ------------------------------------------------------------------------------------ */

/* dst[b] = A[b] (M,K; strides lda0, lda1) x B[b] (K,N; strides ldb0, ldb1).
 * batch_stride_b == 0 broadcasts one B over the batch.
 * Replaces mograd_matmul, kernels/__init__.mojo:616-684.  This is the entry dW^T = X^T dY
 * reaches with A = X^T as a strided view (mograd/grad.mojo:183). */
int mg_matmul(const void* a, const void* b, void* dst, int64_t batch, int64_t M, int64_t N,
              int64_t K, int64_t lda0, int64_t lda1, int64_t ldb0, int64_t ldb1,
              int64_t batch_stride_a, int64_t batch_stride_b, int dtype, mg_stream stream);

/* dst[b] = A[b] (M,K) x B[b]^T with B given as (N,K; strides ldb0, ldb1).
 * Replaces mograd_matmul_bt, kernels/__init__.mojo:687-755.  This is the entry
 * dX = dY W reaches with B = W^T as a strided view. */
int mg_matmul_bt(const void* a, const void* b, void* dst, int64_t batch, int64_t M, int64_t N,
                 int64_t K, int64_t lda0, int64_t lda1, int64_t ldb0, int64_t ldb1,
                 int64_t batch_stride_a, int64_t batch_stride_b, int dtype, mg_stream stream);

/* dst = A x B^T + bias[n].  Replaces mograd_matmul_bias_bt, kernels/__init__.mojo:758-840. */
int mg_matmul_bias_bt(const void* a, const void* b, const void* bias, void* dst, int64_t batch,
                      int64_t M, int64_t N, int64_t K, int64_t lda0, int64_t lda1, int64_t ldb0,
                      int64_t ldb1, int64_t batch_stride_a, int64_t batch_stride_b, int dtype,
                      mg_stream stream);

/* The three Linear gradients for Y(M,N) = X(M,K) W(N,K)^T + b, all contiguous:
 *   dx(M,K) = dY W          (NULL to skip)
 *   dw(N,K) = dY^T X        written directly in W's layout, no transposed view
 *   db(N)   = column sums   (NULL to skip)
 * Covers the graph mograd/grad.mojo:180-187,278-288 emits for a Linear layer. */
int mg_linear_bwd(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db,
                  int64_t M, int64_t N, int64_t K, int dtype, mg_stream stream);

/* Fused forms used by a transformer block.  None has a counterpart in the reference, whose
 * graph runs the matmul and the elementwise op as separate kernels
 * (examples/tinyshakespear/model.mojo:62-64,120-121; mograd/grad.mojo:130-131,180-187).
 * Each gives bit for bit what the separate calls give: for 16-bit types the product is
 * rounded to the storage type before a residual is added.
 *   mg_matmul_bt_add        dst = A x B^T + residual; residual is laid out like dst
 *                           (batch, M, N) and may be dst itself.      MATMUL_BT + ADD
 *   mg_matmul_bias_relu_bt  dst = max(A x B^T + bias, 0).             MATMUL_BIAS_BT + RELU
 *   mg_linear_bwd_fused     mg_linear_bwd with, for dx only:
 *                           x_is_relu_output != 0: dx = (dY W) where x > 0, else 0
 *                                                  (the RELU_GRAD of the layer below);
 *                           dx_accumulate != 0:    dx += that (sum of the input
 *                                                  gradients of layers sharing x). */
int mg_matmul_bt_add(const void* a, const void* b, const void* residual, void* dst, int64_t batch,
                     int64_t M, int64_t N, int64_t K, int64_t lda0, int64_t lda1, int64_t ldb0,
                     int64_t ldb1, int64_t batch_stride_a, int64_t batch_stride_b, int dtype,
                     mg_stream stream);
int mg_matmul_bias_relu_bt(const void* a, const void* b, const void* bias, void* dst, int64_t batch,
                           int64_t M, int64_t N, int64_t K, int64_t lda0, int64_t lda1,
                           int64_t ldb0, int64_t ldb1, int64_t batch_stride_a,
                           int64_t batch_stride_b, int dtype, mg_stream stream);
int mg_linear_bwd_fused(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db,
                        int64_t M, int64_t N, int64_t K, int dx_accumulate, int x_is_relu_output,
                        int dtype, mg_stream stream);

/* dst(outer, inner) = sum over the middle axis of a contiguous (outer, reduce, inner)
 * array.  db = sum over rows is outer=1, reduce=M, inner=N.  Two-stage, no atomics.
 * Replaces mograd_sum_axis for contiguous inputs, kernels/__init__.mojo:1163-1189
 * (kernels/reduce.mojo:137-173). */
int mg_sum_axis(const void* a, void* dst, int64_t outer, int64_t reduce, int64_t inner, int dtype,
                mg_stream stream);

/* dst = upstream where out > 0 else 0, contiguous, n elements.
 * Replaces mograd_relu_grad for contiguous inputs (kernels/elementwise.mojo:66-67). */
int mg_relu_grad(const void* out, const void* upstream, void* dst, int64_t n, int dtype,
                 mg_stream stream);

/* ------------------------------------------------------------------------------------ */
/* The other per-step ops of a transformer block: residual adds, relu, casts, making a   */
/* transposed view contiguous, embedding lookup and its gradient.  Float dtypes only;    */
/* contiguous operands unless strides are passed.                                        */
/* ------------------------------------------------------------------------------------ */

/* dst = a + b over n contiguous elements (dst may alias a or b).
 * Replaces mograd_add, kernels/__init__.mojo:462-471. */
int mg_add(const void* a, const void* b, void* dst, int64_t n, int dtype, mg_stream stream);

/* dst = max(a, 0) over n contiguous elements (dst may alias a).
 * Replaces mograd_relu for a contiguous layout, kernels/__init__.mojo:274-286. */
int mg_relu(const void* a, void* dst, int64_t n, int dtype, mg_stream stream);

/* dst[i] = (out_dtype) a[i], one rounding (nearest even), n contiguous elements.
 * Replaces mograd_cast for a contiguous layout and float types,
 * kernels/__init__.mojo:304-335 (kernels/elementwise.mojo:75-90). */
int mg_cast(const void* a, void* dst, int64_t n, int in_dtype, int out_dtype, mg_stream stream);

/* dst (row-major, contiguous) = the view of `a` with the given shape and element strides
 * (host arrays of `rank` <= 8 entries, strides >= 0, base offset already applied to `a`).
 * Any dtype of the enum.  Replaces mograd_contiguous, kernels/__init__.mojo:338-350. */
int mg_contiguous(const void* a, void* dst, int rank, const int64_t* shape, const int64_t* strides,
                  int dtype, mg_stream stream);

/* The four maps above over strided views: the operands are views of dst's shape (host arrays
 * of `rank` <= 8 extents) with their own element strides, >= 0, 0 along a broadcast axis, base
 * offsets already applied to the pointers; dst is row-major, contiguous, and overlaps neither
 * operand.  Any alignment; views whose innermost axis is contiguous (or constant) and whose
 * rows start on 16-byte boundaries are read 16 bytes at a time, others element by element.
 * The values equal mg_contiguous of each operand followed by the contiguous entry, without
 * the copy (a broadcast bias is never written out).
 * Replace mograd_add_strided (kernels/__init__.mojo:474-487), mograd_relu (:274-286),
 * mograd_relu_grad (:546-560) and mograd_cast (:304-335) for non-contiguous layouts
 * (kernels/strided.mojo:54-114, kernels/elementwise.mojo:75-90). */
int mg_add_strided(const void* a, const void* b, void* dst, int rank, const int64_t* shape,
                   const int64_t* strides_a, const int64_t* strides_b, int dtype, mg_stream stream);
int mg_relu_strided(const void* a, void* dst, int rank, const int64_t* shape, const int64_t* strides,
                    int dtype, mg_stream stream);
int mg_relu_grad_strided(const void* out, const void* upstream, void* dst, int rank,
                         const int64_t* shape, const int64_t* strides_out,
                         const int64_t* strides_upstream, int dtype, mg_stream stream);
int mg_cast_strided(const void* a, void* dst, int rank, const int64_t* shape, const int64_t* strides,
                    int in_dtype, int out_dtype, mg_stream stream);

/* dst(i, :) = src(indices[i], :), i < n_idx; src is (num_rows, row_size) with the given
 * element strides, dst and indices contiguous, idx_dtype MG_I32 or MG_I64 (the reference
 * takes int64 only).  An index outside [0, num_rows) yields a row of zeros (the reference
 * reads out of bounds).  Replaces mograd_gather, kernels/__init__.mojo:132-163
 * (kernels/gather_scatter.mojo:14-38). */
int mg_gather(const void* src, const void* indices, void* dst, int64_t n_idx, int64_t num_rows,
              int64_t row_size, int64_t src_row_stride, int64_t src_col_stride, int idx_dtype,
              int dtype, mg_stream stream);

/* dst(r, :) = sum over i with indices[i] == r of values(i, :); dst is (num_rows, row_size)
 * and is fully written (rows nobody indexes become zero), values is (n_idx, row_size)
 * contiguous.  Rows are added in index order with fp32 accumulation and no atomics, so
 * the result is deterministic (the reference uses atomic adds into a zero-filled
 * buffer).  Indices outside [0, num_rows) are ignored.  Replaces mograd_scatter_add,
 * kernels/__init__.mojo:166-211 (kernels/gather_scatter.mojo:46-71). */
int mg_scatter_add(const void* indices, const void* values, void* dst, int64_t n_idx,
                   int64_t num_rows, int64_t row_size, int idx_dtype, int dtype, mg_stream stream);

/* ------------------------------------------------------------------------------------ */
/* Row softmax, its gradient, argmax.  Contiguous operands, float dtypes, fp32 arithmetic. */
/* ------------------------------------------------------------------------------------ */

/* y = softmax over the last axis of (rows, cols).  Replaces mograd_softmax for a
 * contiguous source, kernels/__init__.mojo:1015-1030 (kernels/softmax.mojo:19-38). */
int mg_softmax(const void* x, void* y, int64_t rows, int64_t cols, int dtype, mg_stream stream);

/* Row softmax over the last axis of a strided view (`rank` >= 1 extents and element strides
 * >= 0, base offset applied to `x`); y is row-major, contiguous.  Same arithmetic as mg_softmax;
 * rows that are contiguous and start on 16-byte boundaries are read 16 bytes at a time.
 * Replaces mograd_softmax_strided, kernels/__init__.mojo:1033-1060 (kernels/softmax.mojo:40-68). */
int mg_softmax_strided(const void* x, void* y, int rank, const int64_t* shape, const int64_t* strides,
                       int dtype, mg_stream stream);

/* dst = y * (upstream - sum over the row of y * upstream).  Replaces mograd_softmax_grad,
 * kernels/__init__.mojo:1062-1090 (kernels/softmax.mojo:76-98). */
int mg_softmax_grad(const void* y, const void* upstream, void* dst, int64_t rows, int64_t cols,
                    int dtype, mg_stream stream);

/* dst(outer, inner) = index along the middle axis of a contiguous (outer, reduce, inner)
 * array of its largest value, stored as a value of `dtype` like the reference does.  A
 * value wins only if strictly greater: ties go to the lowest index, NaN never wins, an
 * all-NaN or empty lane gives 0.  Replaces mograd_argmax_axis for contiguous sources,
 * kernels/__init__.mojo:1269-1301 (kernels/reduce.mojo:208-239). */
int mg_argmax_axis(const void* a, void* dst, int64_t outer, int64_t reduce, int64_t inner, int dtype,
                   mg_stream stream);

/* ------------------------------------------------------------------------------------ */
/* Optimizer updates on flat fp32 arrays (parameters, gradients and moments are fp32 in   */
/* the reference).  One streaming kernel each; in place.                                  */
/* ------------------------------------------------------------------------------------ */

/* One Adam (decoupled_weight_decay == 0: weight decay added to the gradient) or AdamW
 * (!= 0: w scaled by 1 - lr*wd first) update of n parameters, t = step count from 1:
 *   m = m*b1 + g*(1-b1);  v = v*b2 + g*g*(1-b2)
 *   w = w - lr * (m / (1 - b1^t)) / (sqrt(v / (1 - b2^t)) + eps)
 * with the reference's order of operations.  Replaces the elementwise graph that
 * mograd/nn/optim/adam.mojo:6-78 (_adam_step) evaluates per parameter. */
int mg_adam_step(void* w, const void* g, void* m, void* v, int64_t n, float lr, float beta1,
                 float beta2, float eps, float weight_decay, int64_t t,
                 int decoupled_weight_decay, mg_stream stream);

/* w = w - g * lr.  Replaces mograd/nn/optim/sgd.mojo:24-45. */
int mg_sgd_step(void* w, const void* g, int64_t n, float lr, mg_stream stream);

/* ------------------------------------------------------------------------------------ */
/* Deferred second-stage reductions.  No counterpart in the reference, which runs every   */
/* reduction where its graph node is evaluated.                                           */
/*                                                                                        */
/* mg_linear_bwd, mg_layer_norm_bwd_stats(_add) and mg_scatter_add each end in a short     */
/* second kernel that adds fp32 partial results in a fixed order (the K ranges of dW and   */
/* the partial rows of db; the row groups of dgamma/dbeta; the index slabs of the table).  */
/* Nothing in a backward pass reads those sums, so a training step can leave them all to   */
/* one launch at its end.  The `_deferred` forms take the same arguments plus              */
/*   grad_dtype  element type of the parameter gradients this call produces (dw and db;    */
/*               dgamma and dbeta; dst): the tensors' `dtype`, or MG_F32 to get the fp32   */
/*               sums unrounded (fp32 master gradients of a 16-bit layer);                 */
/*   list        an mg_deferred the pending sums are recorded on.                          */
/* They enqueue the first-stage kernels (dx is complete when those are) and return; the    */
/* parameter gradients are valid only after mg_finish_deferred(list, stream), called on    */
/* the same stream, which sums everything on the list in one launch and empties it.  The   */
/* sums use the code of the immediate forms: with grad_dtype == dtype the results are      */
/* bit-identical to them, with MG_F32 they are the same fp32 sums before rounding.  A      */
/* shape whose immediate form has no second stage, or none that can be deferred, is        */
/* computed at once (and converted if grad_dtype differs).  The list keeps the partial     */
/* results' pool blocks until it is finished or destroyed.  One list serves one stream     */
/* and one host thread at a time.                                                          */
/* ------------------------------------------------------------------------------------ */

typedef void* mg_deferred;
int mg_deferred_create(mg_deferred* out);
/* Drops pending sums (their outputs stay unwritten) and frees the list. */
int mg_deferred_destroy(mg_deferred list);
/* Number of sums waiting on the list. */
int mg_deferred_pending(mg_deferred list);
/* Runs every pending sum of `list` in one launch on `stream` and empties the list. */
int mg_finish_deferred(mg_deferred list, mg_stream stream);

/* mg_linear_bwd_fused with dw and db of `grad_dtype`, their sums deferred. */
int mg_linear_bwd_deferred(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db,
                           int64_t M, int64_t N, int64_t K, int dx_accumulate, int x_is_relu_output,
                           int dtype, int grad_dtype, mg_deferred list, mg_stream stream);
/* mg_layer_norm_bwd_stats_add (`residual` may be NULL: mg_layer_norm_bwd_stats) with dgamma
 * and dbeta of `grad_dtype`, their sums deferred. */
int mg_layer_norm_bwd_stats_deferred(const void* dy, const void* x, const void* gamma, const float* mean,
                                     const float* rstd, const void* residual, void* dx, void* dgamma,
                                     void* dbeta, int64_t rows, int64_t cols, int dtype, int grad_dtype,
                                     mg_deferred list, mg_stream stream);
/* A Linear layer's backward continued through the LayerNorm that produced the layer's input:
 * for Y = LN(h) W^T (+ b) with LN(h) = x, given dY,
 *   dW = dY^T x, db = column sums of dY (db may be NULL),
 *   dh = LayerNorm backward of dY W at h with the saved statistics (dx_accumulate != 0: added
 *        to what `dh` holds, the gradient reaching h along a skip connection), dgamma, dbeta,
 * i.e. mg_linear_bwd(dy, x, w, t, dw, db) followed by mg_layer_norm_bwd_stats(_add)(t, h, gamma,
 * mean, rstd, dh, ..) without the (M, K) tensor t = dY W: for 16-bit layers with K == 384 input
 * columns whose backward takes the single launch with 128 x 384 tiles, a tile holds whole rows
 * of t and continues as the LayerNorm backward from LDS; t is rounded to the tensors' type on
 * the way, as storing it would, so only the order of the row and column sums differs from the
 * two separate calls.  Every other shape and dtype runs those two calls with t in a pool block.
 * `list` may be NULL (sums at once, grad_dtype == dtype); otherwise dw, db, dgamma and dbeta
 * are of `grad_dtype` and their sums are deferred as in the `_deferred` forms.  No counterpart
 * in the reference, whose graph evaluates LINEAR_GRAD and the LayerNorm gradient as separate
 * nodes (mograd/grad.mojo:296-344). */
int mg_linear_bwd_layer_norm_bwd(const void* dy, const void* x, const void* w, const void* h,
                                 const void* gamma, const float* mean, const float* rstd, void* dh,
                                 void* dw, void* db, void* dgamma, void* dbeta, int64_t M, int64_t N,
                                 int64_t K, int dx_accumulate, int dtype, int grad_dtype,
                                 mg_deferred list, mg_stream stream);
/* mg_scatter_add with dst of `grad_dtype`, the sum over the index slabs deferred. */
int mg_scatter_add_deferred(const void* indices, const void* values, void* dst, int64_t n_idx,
                            int64_t num_rows, int64_t row_size, int idx_dtype, int dtype, int grad_dtype,
                            mg_deferred list, mg_stream stream);

/* ------------------------------------------------------------------------------------ */
/* Flash attention.  Q, K, V, dQ, dK, dV are BSHD; O and dO are BHSD; mask is            */
/* (B,H,S,S) additive bias in natural-log units, of `dtype`; LSE is (B,H,S) fp32 natural  */
/* log (kernels/attention/generic.mojo:29-35).  dtype in {F32, F16, BF16}.                */
/* causal != 0 with has_bias != 0 is rejected (kernels/__init__.mojo:868-873); with       */
/* has_bias == 0 `mask` is never read and may be any pointer.  1 <= D <= 512 else error   */
/* (kernels/attention/dispatch.mojo:28-29,124-125).                                       */
/* ------------------------------------------------------------------------------------ */

/* Replaces mograd_flash_attn_fwd, kernels/__init__.mojo:848-921. */
int mg_flash_attn_fwd(const void* q, const void* k, const void* v, const void* mask, void* o,
                      float* lse, int64_t B, int64_t S, int64_t H, int64_t D, float scale,
                      int causal, int has_bias, int dtype, mg_stream stream);

/* Replaces mograd_flash_attn_bwd, kernels/__init__.mojo:924-1006. */
int mg_flash_attn_bwd(const void* d_o, const void* o, const void* q, const void* k, const void* v,
                      const void* mask, const float* lse, void* dq, void* dk, void* dv, int64_t B,
                      int64_t S, int64_t H, int64_t D, float scale, int causal, int has_bias,
                      int dtype, mg_stream stream);

/* The same two operations with O and dO laid out (B,S,H,D) like Q, K and V, so that the
 * projection after attention reads O, and the one before it writes dO, without a
 * (B,H,S,D) <-> (B,S,H,D) copy.  LSE stays (B,H,S).  The reference has no such form: its
 * model makes the copy with a CONTIGUOUS node after `transpose(1, 2)`
 * (examples/tinyshakespear/model.mojo:104); results are bit-identical to the standard
 * entry points followed (or preceded) by mg_contiguous. */
int mg_flash_attn_fwd_bshd(const void* q, const void* k, const void* v, const void* mask, void* o,
                           float* lse, int64_t B, int64_t S, int64_t H, int64_t D, float scale,
                           int causal, int has_bias, int dtype, mg_stream stream);
int mg_flash_attn_bwd_bshd(const void* d_o, const void* o, const void* q, const void* k,
                           const void* v, const void* mask, const float* lse, void* dq, void* dk,
                           void* dv, int64_t B, int64_t S, int64_t H, int64_t D, float scale,
                           int causal, int has_bias, int dtype, mg_stream stream);

/* Q, K and V as the three slices of one (B,S,3,H,D) tensor (what a single projection of
 * width 3*H*D writes), dQ, dK, dV likewise in one `dqkv`, O and dO (B,S,H,D), LSE (B,H,S).
 * The gradient with respect to the projection's input and weight is then one product each
 * instead of three.  Same arithmetic and results as the separate-tensor forms; no
 * counterpart in the reference, whose model projects Q, K and V with three Linear layers
 * (examples/tinyshakespear/model.mojo:80-101). */
int mg_flash_attn_fwd_packed(const void* qkv, const void* mask, void* o, float* lse, int64_t B,
                             int64_t S, int64_t H, int64_t D, float scale, int causal, int has_bias,
                             int dtype, mg_stream stream);
int mg_flash_attn_bwd_packed(const void* d_o, const void* o, const void* qkv, const void* mask,
                             const float* lse, void* dqkv, int64_t B, int64_t S, int64_t H,
                             int64_t D, float scale, int causal, int has_bias, int dtype,
                             mg_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* MOGRAD_HIP_H */
