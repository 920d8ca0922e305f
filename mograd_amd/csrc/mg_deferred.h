// Deferred second-stage reductions.
//
// Several entry points end in a short kernel that sums fp32 partial results in a fixed order
// (the K ranges of a split dW with the bias gradient's partial rows, the row groups of
// LayerNorm's dgamma/dbeta, the index slabs of scatter_add).  Nothing in a backward pass reads
// those sums, so a training step can leave them all to one launch at its end: the `_deferred`
// entry points run their main kernels, record the pending sum in an mg_deferred list (which
// keeps the partials' pool blocks alive) and return; mg_finish_deferred sums everything on the
// list with the same code, hence the same order of additions and the same bits, as the
// immediate forms, and may write the sums in fp32 where the immediate forms round to the
// tensors' 16-bit type.
//
// A `_deferred` entry point makes its list current for the calling thread while it runs; the
// places that would launch a second stage ask deferred_current() and hand their work over.
#pragma once

#include <vector>

#include "mg_internal.h"

namespace mg {

enum DeferredKind : int {
  kDeferSplitK = 0,  // K ranges of a split dW, partial tiles in accumulator order
  kDeferBiasRows,    // partial rows of a bias gradient
  kDeferSlab,        // (groups, cols) partials, slab form
  kDeferCw64,        // (groups, cols) partials, 64 / 32 / 16 columns per 256 threads
  kDeferCw32,
  kDeferCw16,
};

// One pending sum, as the finishing kernel takes it (passed by value in the kernel arguments).
struct DeferredJob {
  const float* part;
  void* out;
  int64_t slice;  // kDeferSplitK: floats per K range
  int kind;
  int out_dtype;
  int rows;    // kDeferSplitK: rows of dW to write
  int cols;    // kDeferSplitK: columns of dW; others: number of outputs
  int groups;  // partial slices to add
  int block_end;  // in the launch: one past this job's last 1024-thread workgroup; on the list: its workgroups
};

struct DeferredList {
  std::vector<DeferredJob> jobs;
  std::vector<void*> held;  // pool blocks of the partials, released by the finishing call
  // While a `_deferred` entry point runs: the element type its outputs are written in, and the
  // substitutions (from, to) of output pointers made for it (see DeferredScope).
  int out_dtype = MG_F32;
  std::vector<std::pair<void*, void*>> redirect;

  void* target(void* out) const {
    for (const auto& r : redirect)
      if (r.first == out) return r.second;
    return out;
  }
  void push(int kind, const float* part, void* out, int64_t slice, int rows, int cols, int groups, int64_t blocks) {
    jobs.push_back(DeferredJob{part, target(out), slice, kind, out_dtype, rows, cols, groups, static_cast<int>(blocks)});
  }
  // Takes over the pool block of `s`: it now lives until the list is finished.
  void hold(Scratch& s) {
    if (void* p = s.detach()) held.push_back(p);
  }
};

// The list of the `_deferred` entry point running on this thread, or null.
DeferredList* deferred_current();
void deferred_set_current(DeferredList* list);

// Workgroups of 1024 threads that a (groups, cols) sum of the given form needs.
inline int64_t deferred_column_blocks(int variant, int64_t cols) {
  return variant == 0 ? ceil_div(cols, 32) : ceil_div(ceil_div(cols, variant), 4);
}

// Makes `list` current for one entry point.  An output whose element type differs from the
// tensors' (fp32 gradients of a 16-bit layer) is replaced by a scratch buffer of the tensors'
// type for the duration: whatever part of the call defers its sum is redirected to write the
// real output in `out_dtype`; outputs that the call produced at once are converted afterwards
// (finish()).
class DeferredScope {
 public:
  DeferredScope(DeferredList* list, int dtype, int out_dtype) : list_(list), dtype_(dtype), out_dtype_(out_dtype) {
    list_->out_dtype = out_dtype;
    list_->redirect.clear();
    deferred_set_current(list_);
  }
  ~DeferredScope() {
    deferred_set_current(nullptr);
    list_->redirect.clear();
    for (auto& t : temps_) pool_release(t.tmp);
  }
  // The pointer to hand to the kernels in place of `out` (numel elements).
  int substitute(void* out, int64_t numel, void** use) {
    *use = out;
    if (!out || out_dtype_ == dtype_) return MG_OK;
    void* tmp = nullptr;
    MG_TRY(pool_take(&tmp, numel * dtype_size(dtype_)));
    temps_.push_back(Temp{tmp, out, numel, list_->jobs.size()});
    list_->redirect.emplace_back(tmp, out);
    *use = tmp;
    return MG_OK;
  }
  // After the entry point's work is enqueued: converts the substituted outputs that no
  // deferred job took over.
  int finish(hipStream_t stream) {
    for (const auto& t : temps_) {
      bool deferred = false;
      for (size_t j = t.first_job; j < list_->jobs.size(); ++j) deferred |= list_->jobs[j].out == t.real;
      if (!deferred) MG_TRY(mg_cast(t.tmp, t.real, t.numel, dtype_, out_dtype_, stream));
    }
    return MG_OK;
  }

 private:
  struct Temp {
    void* tmp;
    void* real;
    int64_t numel;
    size_t first_job;
  };
  DeferredList* list_;
  int dtype_, out_dtype_;
  std::vector<Temp> temps_;
};

// Argument checks shared by the `_deferred` entry points.
inline int deferred_check(const char* who, void* list, int dtype, int grad_dtype) {
  if (!list) return fail(MG_ERR_INVALID, "%s: null deferred list", who);
  if (!is_float_dtype(grad_dtype) || (grad_dtype != dtype && grad_dtype != MG_F32))
    return fail(MG_ERR_INVALID, "%s: grad_dtype must be the tensors' dtype or float32, got %s", who, dtype_name(grad_dtype));
  return MG_OK;
}

}  // namespace mg
