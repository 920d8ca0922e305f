// The list of deferred second-stage reductions and the one launch that finishes them.
#include "gemm_impl.h"
#include "mg_deferred.h"
#include "mg_rows.h"

namespace mg {

static thread_local DeferredList* tls_deferred = nullptr;
DeferredList* deferred_current() { return tls_deferred; }
void deferred_set_current(DeferredList* list) { tls_deferred = list; }

// Jobs of one launch, passed by value in the kernel arguments (4 KB at most).
constexpr int kDeferredMaxJobs = 64;
struct DeferredTable {
  int count;
  DeferredJob job[kDeferredMaxJobs];
};

// LDS of a finishing workgroup: the largest of the forms' needs.
constexpr int kDeferredLdsBytes = kSlabLdsFloats * 4 > 4096 ? kSlabLdsFloats * 4 : 4096;

template <typename OutT>
__device__ __forceinline__ void deferred_run(char* lds, const DeferredJob& j, int local_block) {
  OutT* out = static_cast<OutT*>(j.out);
  const int sub = threadIdx.x / 256, tid = threadIdx.x % 256;
  switch (j.kind) {
    case kDeferSplitK:
      // a thread sums four consecutive values of a partial tile over the K ranges
      gemm_splitk_reduce_group<OutT, false, true, true>(static_cast<int64_t>(local_block) * 1024 + threadIdx.x, j.part,
                                                  static_cast<const OutT*>(nullptr), out, j.slice, j.slice, j.groups,
                                                  j.cols, GemmEpilogue<OutT>{nullptr, nullptr, 0}, j.rows,
                                                  (j.cols + kGemmBN - 1) / kGemmBN);
      break;
    case kDeferBiasRows:
      linear_bwd_db_block<OutT>(reinterpret_cast<float*>(lds) + sub * 256, tid, local_block * 4 + sub, j.part, out,
                                j.groups, j.cols);
      break;
    case kDeferSlab:
      reduce_partials_slab_block<OutT>(reinterpret_cast<float*>(lds), local_block, j.part, out, j.groups, j.cols);
      break;
    case kDeferCw64:
      reduce_partials_cw_block<OutT, 64>(reinterpret_cast<float*>(lds) + sub * 256, tid,
                                         static_cast<int64_t>(local_block) * 4 + sub, j.part, out, j.groups, j.cols);
      break;
    case kDeferCw32:
      reduce_partials_cw_block<OutT, 32>(reinterpret_cast<float*>(lds) + sub * 256, tid,
                                         static_cast<int64_t>(local_block) * 4 + sub, j.part, out, j.groups, j.cols);
      break;
    default:
      reduce_partials_cw_block<OutT, 16>(reinterpret_cast<float*>(lds) + sub * 256, tid,
                                         static_cast<int64_t>(local_block) * 4 + sub, j.part, out, j.groups, j.cols);
      break;
  }
}

// Workgroup b serves the job whose range of workgroups [block_end of its predecessor,
// block_end) holds b; every workgroup is of one job and one form, so the barriers inside the
// forms are reached by all of its threads.
__global__ __launch_bounds__(1024) void deferred_finish_kernel(const DeferredTable tab) {
  __shared__ __attribute__((aligned(16))) char lds[kDeferredLdsBytes];
  const int b = blockIdx.x;
  int lo = 0, hi = tab.count - 1;  // first job with block_end > b
  while (lo < hi) {
    const int mid = (lo + hi) / 2;
    if (tab.job[mid].block_end > b) hi = mid;
    else lo = mid + 1;
  }
  const DeferredJob& j = tab.job[lo];
  const int local_block = b - (lo > 0 ? tab.job[lo - 1].block_end : 0);
  switch (j.out_dtype) {
    case MG_F32: deferred_run<float>(lds, j, local_block); break;
    case MG_F16: deferred_run<f16_t>(lds, j, local_block); break;
    default: deferred_run<bf16_t>(lds, j, local_block); break;
  }
}

static int deferred_release(DeferredList* dl) {
  int rc = MG_OK;
  for (void* p : dl->held) {
    const int r = pool_release(p);
    if (r != MG_OK) rc = r;
  }
  dl->held.clear();
  dl->jobs.clear();
  return rc;
}

static int deferred_finish(DeferredList* dl, hipStream_t stream) {
  size_t at = 0;
  while (at < dl->jobs.size()) {
    DeferredTable tab;
    tab.count = 0;
    int64_t blocks = 0;
    while (at < dl->jobs.size() && tab.count < kDeferredMaxJobs) {
      DeferredJob j = dl->jobs[at];
      const int64_t n = j.block_end;  // held the job's own count until now
      if (blocks + n > 0x7fffffffLL) {
        if (tab.count == 0) return fail(MG_ERR_INVALID, "finish_deferred: a single sum exceeds the launch grid");
        break;
      }
      ++at;
      if (n <= 0) continue;
      blocks += n;
      j.block_end = static_cast<int>(blocks);
      tab.job[tab.count++] = j;
    }
    if (tab.count == 0) continue;
    hipLaunchKernelGGL(deferred_finish_kernel, dim3(static_cast<unsigned>(blocks)), dim3(1024), 0, stream, tab);
    MG_LAUNCH_CHECK();
  }
  return MG_OK;
}

}  // namespace mg

extern "C" {

int mg_deferred_create(mg_deferred* out) {
  if (!out) return mg::fail(MG_ERR_INVALID, "deferred_create: null output pointer");
  *out = new mg::DeferredList();
  return MG_OK;
}

int mg_deferred_destroy(mg_deferred list) {
  if (!list) return MG_OK;
  mg::DeferredList* dl = static_cast<mg::DeferredList*>(list);
  const int rc = mg::deferred_release(dl);  // pending sums are dropped
  delete dl;
  return rc;
}

int mg_deferred_pending(mg_deferred list) {
  return list ? static_cast<int>(static_cast<mg::DeferredList*>(list)->jobs.size()) : 0;
}

int mg_finish_deferred(mg_deferred list, mg_stream stream) {
  if (!list) return mg::fail(MG_ERR_INVALID, "finish_deferred: null deferred list");
  mg::DeferredList* dl = static_cast<mg::DeferredList*>(list);
  const int rc = mg::deferred_finish(dl, mg::to_stream(stream));
  const int rc2 = mg::deferred_release(dl);
  return rc != MG_OK ? rc : rc2;
}

}  // extern "C"
