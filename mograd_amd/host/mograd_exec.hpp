// C++ host side of the backward hot path: the reference's kernel-dispatch surface restated
// over libmograd_hip.so for a compiled caller.
//
// The reference's scheduler maps an op node to a `BoundExecFn(node, inputs, device) ->
// List[AnyBuffer]` (mograd/scheduler.mojo:13-15) whose body turns layouts into a kernel call
// (mograd/runtime/gpu/kernels/dispatch.mojo).  This header restates that surface with the
// same names, argument derivations and error conditions; it contains no arithmetic, every
// result comes from the C ABI declared in mograd_hip.h.  It is the C++ twin of
// mograd_amd/runtime.py (which the Python tests drive) and what a Mojo binding of the
// library would look like line for line:
//
//     Layout            shape + element strides + base offset      mograd/layout.mojo:15-28
//     Device            library handle, per-name symbol cache,     mograd/device_ctx.mojo:25-113
//                       one in-order stream
//     AnyBuffer         typed device allocation from the pool      mograd/buffer.mojo:135-214
//     OpRef             (op_type, layout, dtype, srcs, attrs)      mograd/op.mojo:124-185
//     scheduler_rules   op type -> exec function                   mograd/runtime/__init__.mojo:113-167
//
// Header-only, C++17, needs only libdl.  The library is found through $MOGRAD_HIP_SO, as the
// reference finds its own through $MOGRAD_SO (device_ctx.mojo:47-51); a missing library is
// an error, there is no fallback.
#pragma once

#include <dlfcn.h>

#include <cstdint>
#include <cstdlib>
#include <map>
#include <optional>
#include <memory>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "mograd_hip.h"

namespace mograd {

// What the reference raises as a Mojo `Error`: the status code of the C ABI and its message.
struct Error : std::runtime_error {
  int code;
  Error(int c, const std::string& msg) : std::runtime_error(msg), code(c) {}
};

using DType = int;  // mg_dtype codes
constexpr DType float32 = MG_F32, float16 = MG_F16, bfloat16 = MG_BF16, int32 = MG_I32, int64 = MG_I64;

inline int dtype_size(DType d) {
  switch (d) {
    case MG_F32: case MG_I32: return 4;
    case MG_F16: case MG_BF16: return 2;
    case MG_I64: return 8;
    default: return 0;
  }
}

// ---- Layout (mograd/layout.mojo) -------------------------------------------------------------

class Layout {
 public:
  Layout() = default;
  Layout(std::vector<int64_t> shape) : dims_(std::move(shape)), strides_(row_major(dims_)) {}  // NOLINT: implicit on purpose
  Layout(std::initializer_list<int64_t> shape) : Layout(std::vector<int64_t>(shape)) {}
  Layout(std::vector<int64_t> shape, std::vector<int64_t> strides, int64_t base_offset = 0)
      : dims_(std::move(shape)), strides_(std::move(strides)), base_offset_(base_offset) {
    if (dims_.size() != strides_.size()) throw Error(MG_ERR_INVALID, "strides rank differs from shape rank");
  }

  int rank() const { return static_cast<int>(dims_.size()); }
  const std::vector<int64_t>& shape() const { return dims_; }
  const std::vector<int64_t>& stride() const { return strides_; }
  int64_t shape(int i) const { return dims_.at(i); }
  int64_t stride(int i) const { return strides_.at(i); }
  int64_t base_offset() const { return base_offset_; }
  int64_t numel() const {
    int64_t n = 1;
    for (int64_t d : dims_) n *= d;
    return n;
  }
  bool is_contiguous() const { return strides_ == row_major(dims_); }  // layout.mojo:210-212
  Layout as_contiguous() const { return Layout(dims_); }               // layout.mojo:238-240

  // layout.mojo:214-236: every batch dim above the last three folds into one stride.
  bool batch_dims_collapsible() const {
    for (int i = rank() - 4; i >= 0; --i)
      if (strides_[i] != dims_[i + 1] * strides_[i + 1]) return false;
    return true;
  }

  // layout.mojo:287-298: (outer, reduce, inner) extents around `axis`.
  void reduce_dims(int axis, int64_t& outer, int64_t& reduce, int64_t& inner) const {
    const int ax = axis < 0 ? axis + rank() : axis;
    if (ax < 0 || ax >= rank())
      throw Error(MG_ERR_INVALID, "axis " + std::to_string(axis) + " out of range for rank " + std::to_string(rank()));
    reduce = dims_[ax];
    inner = 1;
    for (int i = ax + 1; i < rank(); ++i) inner *= dims_[i];
    outer = (reduce != 0 && inner != 0) ? numel() / (reduce * inner) : 0;
  }

  Layout transpose(int dim0 = -2, int dim1 = -1) const {  // layout.mojo:435-452
    const int d0 = ((dim0 % rank()) + rank()) % rank(), d1 = ((dim1 % rank()) + rank()) % rank();
    Layout out = *this;
    std::swap(out.dims_[d0], out.dims_[d1]);
    std::swap(out.strides_[d0], out.strides_[d1]);
    return out;
  }

  Layout slice_axis(int axis, int64_t start, int64_t stop, int64_t step = 1) const {  // layout.mojo:321-340
    const int ax = ((axis % rank()) + rank()) % rank();
    Layout out = *this;
    const int64_t extent = (stop - start + step - 1) / step;
    out.dims_[ax] = extent > 0 ? extent : 0;
    out.strides_[ax] = strides_[ax] * step;
    out.base_offset_ = base_offset_ + start * strides_[ax];
    return out;
  }

 private:
  static std::vector<int64_t> row_major(const std::vector<int64_t>& shape) {
    std::vector<int64_t> st(shape.size(), 1);
    for (int i = static_cast<int>(shape.size()) - 2; i >= 0; --i) st[i] = st[i + 1] * shape[i + 1];
    return st;
  }
  std::vector<int64_t> dims_, strides_;
  int64_t base_offset_ = 0;
};

// ---- Device (mograd/device_ctx.mojo:25-113) ----------------------------------------------------

// One GPU, the library handle, one in-order stream.  Symbols are looked up by name and cached,
// as the reference's `Device.get_function` does per kernel call (device_ctx.mojo:107-113).
class Device {
 public:
  explicit Device(int index = 0, const char* so_path = nullptr) {
    const char* path = so_path ? so_path : std::getenv("MOGRAD_HIP_SO");
    if (!path || !*path) throw Error(MG_ERR_INVALID, "MOGRAD_HIP_SO is not set: the HIP library is required, there is no fallback");
    handle_ = dlopen(path, RTLD_NOW | RTLD_LOCAL | RTLD_NODELETE);
    if (!handle_) throw Error(MG_ERR_INVALID, std::string("cannot load ") + path + ": " + dlerror());
    check(fn<decltype(&::mg_init)>("mg_init")(index));
    check(fn<decltype(&::mg_stream_create)>("mg_stream_create")(&stream_));
  }
  ~Device() {
    if (stream_) {
      fn<decltype(&::mg_stream_sync)>("mg_stream_sync")(stream_);
      fn<decltype(&::mg_stream_destroy)>("mg_stream_destroy")(stream_);
    }
  }
  Device(const Device&) = delete;
  Device& operator=(const Device&) = delete;

  // Typed pointer to the exported symbol `name`; throws if the library does not export it.
  template <typename Fn>
  Fn fn(const char* name) {
    auto it = cache_.find(name);
    if (it == cache_.end()) {
      void* sym = dlsym(handle_, name);
      if (!sym) throw Error(MG_ERR_UNSUPPORTED, std::string("library does not export ") + name);
      it = cache_.emplace(name, sym).first;
    }
    return reinterpret_cast<Fn>(it->second);
  }

  // A non-zero status becomes an Error carrying the library's message for this thread.
  void check(int rc) {
    if (rc != MG_OK) throw Error(rc, fn<decltype(&::mg_last_error)>("mg_last_error")());
  }

  mg_stream stream() const { return stream_; }
  // While set (DeferredSums below), the exec functions of LINEAR_GRAD, LAYER_NORM_STATS_GRAD(_ADD)
  // and SCATTER_ADD leave their second-stage sums on this list.
  mg_deferred pending = nullptr;
  void synchronize() { check(fn<decltype(&::mg_stream_sync)>("mg_stream_sync")(stream_)); }  // ctx.synchronize()
  void empty_cache() { check(fn<decltype(&::mg_pool_empty_cache)>("mg_pool_empty_cache")()); }
  mg_pool_stats memory_stats() {
    mg_pool_stats st{};
    check(fn<decltype(&::mg_pool_get_stats)>("mg_pool_get_stats")(&st));
    return st;
  }

 private:
  void* handle_ = nullptr;
  mg_stream stream_ = nullptr;
  std::unordered_map<std::string, void*> cache_;
};

// Calls exported function `name` with the prototype mograd_hip.h declares for it.
#define MOGRAD_CALL(device, name, ...) (device).check((device).fn<decltype(&::name)>(#name)(__VA_ARGS__))

// ---- AnyBuffer (mograd/buffer.mojo:135-214, mograd/memory.mojo:199-239) --------------------------

// One pooled allocation; goes back to the pool's free lists when the last view dies.
class Storage {
 public:
  Storage(Device& device, int64_t nbytes) : device_(device), nbytes_(nbytes) {
    MOGRAD_CALL(device_, mg_pool_alloc, &ptr_, nbytes);
  }
  ~Storage() {
    if (ptr_) device_.fn<decltype(&::mg_pool_free)>("mg_pool_free")(ptr_);
  }
  Storage(const Storage&) = delete;
  Storage& operator=(const Storage&) = delete;
  void* ptr() const { return ptr_; }
  int64_t nbytes() const { return nbytes_; }
  Device& device() const { return device_; }

 private:
  Device& device_;
  void* ptr_ = nullptr;
  int64_t nbytes_;
};

class AnyBuffer {
 public:
  AnyBuffer() = default;
  static bool supports(DType d) { return dtype_size(d) != 0; }

  static AnyBuffer create(DType dtype, Device& device, int64_t numel) {
    if (!supports(dtype)) throw Error(MG_ERR_INVALID, "Unsupported dtype: " + std::to_string(dtype));
    AnyBuffer b;
    b.storage_ = std::make_shared<Storage>(device, numel * dtype_size(dtype));
    b.dtype_ = dtype;
    b.numel_ = numel;
    return b;
  }
  // Uploads `numel` elements already in the buffer's storage format.
  static AnyBuffer from_host(Device& device, const void* host, int64_t numel, DType dtype) {
    AnyBuffer b = create(dtype, device, numel);
    MOGRAD_CALL(device, mg_copy_to_device, b.data_ptr(), host, numel * dtype_size(dtype), device.stream());
    return b;
  }
  // Synchronous download of the viewed elements as stored (the view must be contiguous).
  void to_host(void* host) const {
    Device& d = storage_->device();
    MOGRAD_CALL(d, mg_copy_to_host, host, data_ptr(), numel_ * dtype_size(dtype_), d.stream());
  }

  // Raw device pointer including the view's base offset (buffer.mojo:196-203).
  void* data_ptr() const { return static_cast<char*>(storage_->ptr()) + offset_elems_ * dtype_size(dtype_); }
  DType dtype() const { return dtype_; }
  int64_t numel() const { return numel_; }
  int64_t offset_elems() const { return offset_elems_; }
  // Shares storage; the element count and base offset come from `layout`.
  AnyBuffer view(const Layout& layout) const {
    AnyBuffer b = *this;
    b.numel_ = layout.numel();
    b.offset_elems_ = layout.base_offset();
    return b;
  }

 private:
  std::shared_ptr<Storage> storage_;
  DType dtype_ = float32;
  int64_t numel_ = 0, offset_elems_ = 0;
};

// ---- Op nodes (mograd/op.mojo:124-185) -------------------------------------------------------------

// Just enough of an op node for the exec functions: its own layout and dtype, its sources'
// layouts and dtypes, and its attributes.
struct OpRef {
  std::string op_type;
  Layout node_layout;
  DType node_dtype = float32;
  std::vector<OpRef> srcs;
  std::map<std::string, double> node_attrs;

  const Layout& layout() const { return node_layout; }
  DType dtype() const { return node_dtype; }
  int64_t numel() const { return node_layout.numel(); }
  const OpRef& src(int i) const { return srcs.at(i); }
  int64_t shape(int i) const { return node_layout.shape(i); }
  bool has_attr(const char* k) const { return node_attrs.count(k) != 0; }
  double attr(const char* k) const {
    auto it = node_attrs.find(k);
    if (it == node_attrs.end()) throw Error(MG_ERR_INVALID, std::string("missing attribute ") + k);
    return it->second;
  }
  static OpRef leaf(const Layout& layout, DType dtype = float32) { return OpRef{"BUFFER", layout, dtype, {}, {}}; }
};

// Value of a FLASH_ATTN / FLASH_ATTN_GRAD node's "layout" attribute when O and dO are (B, S, H, D).
constexpr double kLayoutBshd = 1.0;

using Buffers = std::vector<AnyBuffer>;
using BoundExecFn = Buffers (*)(const OpRef& node, const Buffers& inputs, Device& device);

namespace detail {

inline void require_float(DType d, const char* who) {  // dispatch_dtype[float_only=True], dispatch.mojo:564-576
  if (d != float32 && d != float16 && d != bfloat16) throw Error(MG_ERR_INVALID, std::string(who) + ": unsupported dtype");
}

// The first `count` operands as contiguous buffers.  The reference reads strided views
// element by element inside each kernel (kernels/strided.mojo).  add, relu, relu_grad, cast and
// softmax have strided entries of their own; for the kernels that use this helper a strided operand
// is first copied row-major with mg_contiguous and the contiguous kernel runs on the copy.
// Whether the first `count` operands can take a flat kernel: contiguous, and starting on the
// 16-byte boundary those kernels read from (a view into the middle of a buffer may not).
inline bool flat(const OpRef& node, const Buffers& inputs, int count) {
  for (int i = 0; i < count; ++i)
    if (!node.src(i).layout().is_contiguous() || reinterpret_cast<uintptr_t>(inputs[i].data_ptr()) % 16 != 0) return false;
  return true;
}

inline Buffers materialise(const OpRef& node, const Buffers& inputs, Device& device, int count) {
  Buffers out = inputs;
  for (int i = 0; i < count; ++i) {
    const Layout& l = node.src(i).layout();
    if (l.is_contiguous()) continue;
    AnyBuffer tmp = AnyBuffer::create(node.src(i).dtype(), device, l.numel());
    MOGRAD_CALL(device, mg_contiguous, inputs[i].data_ptr(), tmp.data_ptr(), l.rank(), l.shape().data(), l.stride().data(),
                node.src(i).dtype(), device.stream());
    out[i] = tmp;
  }
  return out;
}

struct MatmulDims {
  int64_t batch, M, K, lda0, lda1, ldb0, ldb1, bsa, bsb;
};
// kernels/__init__.mojo:629-644,700-715,774-786
inline MatmulDims matmul_dims(const Layout& la, const Layout& lb, int64_t N, bool b_is_nk, const char* who) {
  const int ra = la.rank(), rb = lb.rank();
  if (!(la.batch_dims_collapsible() && lb.batch_dims_collapsible()))
    throw Error(MG_ERR_INVALID,
                std::string(who) + ": received non-collapsible batch dims, expected op.mojo to materialise these first");
  MatmulDims d;
  d.M = la.shape(ra - 2);
  d.K = la.shape(ra - 1);
  d.lda0 = la.stride(ra - 2);
  d.lda1 = la.stride(ra - 1);
  d.ldb0 = lb.stride(rb - 2);
  d.ldb1 = lb.stride(rb - 1);
  d.batch = (d.M != 0 && d.K != 0) ? la.numel() / (d.M * d.K) : 0;
  d.bsa = ra >= 3 ? la.stride(ra - 3) : d.M * d.K;
  d.bsb = rb >= 3 ? lb.stride(rb - 3) : (b_is_nk ? N * d.K : d.K * N);
  return d;
}

}  // namespace detail

// ---- Exec functions (BoundExecFn bodies) --------------------------------------------------------------

// LAYER_NORM[x, gamma, beta]{eps}.  dispatch.mojo:294-314.
inline Buffers layer_norm_fwd(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& x = node.src(0).layout();
  const int64_t cols = x.shape(x.rank() - 1), rows = x.numel() / cols;
  detail::require_float(node.dtype(), "layer_norm_fwd");
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_layer_norm_fwd, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), out.data_ptr(),
              rows, cols, static_cast<float>(node.attr("eps")), node.dtype(), device.stream());
  return {out};
}

// LAYER_NORM_GRAD[dy, x, gamma]{eps} -> [dx, dgamma, dbeta].  dispatch.mojo:332-358.
inline Buffers layer_norm_bwd(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& x = node.src(1).layout();
  const Layout& gamma = node.src(2).layout();
  const int64_t cols = x.shape(x.rank() - 1), rows = x.numel() / cols;
  detail::require_float(node.dtype(), "layer_norm_bwd");
  AnyBuffer dx = AnyBuffer::create(node.dtype(), device, x.numel());
  AnyBuffer dgamma = AnyBuffer::create(node.dtype(), device, gamma.numel());
  AnyBuffer dbeta = AnyBuffer::create(node.dtype(), device, gamma.numel());
  MOGRAD_CALL(device, mg_layer_norm_bwd, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), dx.data_ptr(),
              dgamma.data_ptr(), dbeta.data_ptr(), rows, cols, static_cast<float>(node.attr("eps")), node.dtype(),
              device.stream());
  return {dx, dgamma, dbeta};
}

// FLASH_ATTN[Q, K, V, mask]{scale, is_causal, has_bias} -> [O (BHSD), LSE (BHS f32)].
// dispatch.mojo:380-415: B,S,H,D from the BSHD Q layout; has_bias defaults to true.
inline Buffers flash_attn_fwd_sched(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& q = node.src(0).layout();
  const int64_t B = q.shape(0), S = q.shape(1), H = q.shape(2), D = q.shape(3);
  const bool is_causal = node.attr("is_causal") != 0;
  const bool has_bias = node.has_attr("has_bias") ? node.attr("has_bias") != 0 : true;
  detail::require_float(node.dtype(), "flash_attn_fwd");
  AnyBuffer dst = AnyBuffer::create(node.dtype(), device, node.numel());
  AnyBuffer lse = AnyBuffer::create(float32, device, B * H * S);
  // {layout: kLayoutBshd} (set by fuse_attention_output_layout): O is written (B, S, H, D) like Q
  if (node.has_attr("layout") && node.attr("layout") == kLayoutBshd)
    MOGRAD_CALL(device, mg_flash_attn_fwd_bshd, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                inputs[3].data_ptr(), dst.data_ptr(), static_cast<float*>(lse.data_ptr()), B, S, H, D,
                static_cast<float>(node.attr("scale")), is_causal, has_bias, node.dtype(), device.stream());
  else
    MOGRAD_CALL(device, mg_flash_attn_fwd, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                inputs[3].data_ptr(), dst.data_ptr(), static_cast<float*>(lse.data_ptr()), B, S, H, D,
                static_cast<float>(node.attr("scale")), is_causal, has_bias, node.dtype(), device.stream());
  return {dst, lse};
}

// FLASH_ATTN_GRAD[dO, O, Q, K, V, mask, LSE] -> [dQ, dK, dV].
// dispatch.mojo:441-481: has_bias defaults to `not is_causal`.
inline Buffers flash_attn_bwd_sched(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& q = node.src(2).layout();
  const int64_t B = q.shape(0), S = q.shape(1), H = q.shape(2), D = q.shape(3);
  const bool is_causal = node.attr("is_causal") != 0;
  const bool has_bias = node.has_attr("has_bias") ? node.attr("has_bias") != 0 : !is_causal;
  detail::require_float(node.dtype(), "flash_attn_bwd");
  AnyBuffer dq = AnyBuffer::create(node.dtype(), device, q.numel());
  AnyBuffer dk = AnyBuffer::create(node.dtype(), device, q.numel());
  AnyBuffer dv = AnyBuffer::create(node.dtype(), device, q.numel());
  if (node.has_attr("layout") && node.attr("layout") == kLayoutBshd)
    MOGRAD_CALL(device, mg_flash_attn_bwd_bshd, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                inputs[3].data_ptr(), inputs[4].data_ptr(), inputs[5].data_ptr(),
                static_cast<const float*>(inputs[6].data_ptr()), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, S, H, D,
                static_cast<float>(node.attr("scale")), is_causal, has_bias, node.dtype(), device.stream());
  else
    MOGRAD_CALL(device, mg_flash_attn_bwd, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                inputs[3].data_ptr(), inputs[4].data_ptr(), inputs[5].data_ptr(),
                static_cast<const float*>(inputs[6].data_ptr()), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, S, H, D,
                static_cast<float>(node.attr("scale")), is_causal, has_bias, node.dtype(), device.stream());
  return {dq, dk, dv};
}

// CROSS_ENTROPY[logits, labels] -> (1,).  runtime/__init__.mojo:530-533: contiguous operands
// take the flat kernel, anything else the strided one.
inline Buffers cross_entropy(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& la = node.src(0).layout();
  const Layout& lb = node.src(1).layout();
  detail::require_float(node.dtype(), "cross_entropy");
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  const int64_t C = la.shape(la.rank() - 1), N = la.numel() / C;
  if (la.is_contiguous() && lb.is_contiguous())
    MOGRAD_CALL(device, mg_cross_entropy, inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), N, C, node.dtype(),
                device.stream());
  else
    MOGRAD_CALL(device, mg_cross_entropy_strided, inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), la.rank(),
                la.shape().data(), la.stride().data(), lb.stride().data(), node.dtype(), device.stream());
  return {out};
}

// CROSS_ENTROPY_GRAD[logits, labels, upstream].  runtime/__init__.mojo:563-580.
inline Buffers cross_entropy_grad(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& la = node.src(0).layout();
  const Layout& lb = node.src(1).layout();
  detail::require_float(node.dtype(), "cross_entropy_grad");
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  const int64_t C = la.shape(la.rank() - 1), N = la.numel() / C;
  if (la.is_contiguous() && lb.is_contiguous())
    MOGRAD_CALL(device, mg_cross_entropy_grad, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                out.data_ptr(), N, C, node.dtype(), device.stream());
  else
    MOGRAD_CALL(device, mg_cross_entropy_grad_strided, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                out.data_ptr(), la.rank(), la.shape().data(), la.stride().data(), lb.stride().data(), node.dtype(),
                device.stream());
  return {out};
}

// MATMUL[A (.., M, K), B (.., K, N)].  dispatch.mojo:227-244.
inline Buffers matmul(const OpRef& node, const Buffers& inputs, Device& device) {
  const int64_t N = node.shape(node.layout().rank() - 1);
  const auto d = detail::matmul_dims(node.src(0).layout(), node.src(1).layout(), N, false, "matmul");
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_matmul, inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), d.batch, d.M, N, d.K, d.lda0,
              d.lda1, d.ldb0, d.ldb1, d.bsa, d.bsb, node.dtype(), device.stream());
  return {out};
}

// MATMUL_BT[A (.., M, K), B (.., N, K)] = A B^T.  dispatch.mojo:227-244.
inline Buffers matmul_t(const OpRef& node, const Buffers& inputs, Device& device) {
  const int64_t N = node.shape(node.layout().rank() - 1);
  const auto d = detail::matmul_dims(node.src(0).layout(), node.src(1).layout(), N, true, "matmul");
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_matmul_bt, inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), d.batch, d.M, N, d.K,
              d.lda0, d.lda1, d.ldb0, d.ldb1, d.bsa, d.bsb, node.dtype(), device.stream());
  return {out};
}

// MATMUL_BIAS_BT[A, B (N, K), bias (N)] = A B^T + bias.  dispatch.mojo:260-278.
inline Buffers matmul_bias_bt(const OpRef& node, const Buffers& inputs, Device& device) {
  const int64_t N = node.shape(node.layout().rank() - 1);
  const auto d = detail::matmul_dims(node.src(0).layout(), node.src(1).layout(), N, true, "matmul_bias");
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_matmul_bias_bt, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), out.data_ptr(),
              d.batch, d.M, N, d.K, d.lda0, d.lda1, d.ldb0, d.ldb1, d.bsa, d.bsb, node.dtype(), device.stream());
  return {out};
}

// SUM{axis}.  runtime/__init__.mojo:390-393, dispatch.mojo:196-212.  Only the axis form is on
// this path (db = dY.sum(0)).
inline Buffers sum(const OpRef& node, const Buffers& inputs, Device& device) {
  if (!node.has_attr("axis")) throw Error(MG_ERR_UNSUPPORTED, "sum: the full reduction is outside the backward hot path");
  const Buffers in = detail::materialise(node, inputs, device, 1);
  int64_t outer, reduce, inner;
  node.src(0).layout().reduce_dims(static_cast<int>(node.attr("axis")), outer, reduce, inner);
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_sum_axis, in[0].data_ptr(), out.data_ptr(), outer, reduce, inner, node.dtype(), device.stream());
  return {out};
}

// RELU_GRAD[relu_out, upstream].  runtime/__init__.mojo:351-352.
inline Buffers relu_grad(const OpRef& node, const Buffers& in, Device& device) {
  const Layout &la = node.src(0).layout(), &lb = node.src(1).layout();
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  if (detail::flat(node, in, 2))
    MOGRAD_CALL(device, mg_relu_grad, in[0].data_ptr(), in[1].data_ptr(), out.data_ptr(), node.numel(), node.dtype(),
                device.stream());
  else
    MOGRAD_CALL(device, mg_relu_grad_strided, in[0].data_ptr(), in[1].data_ptr(), out.data_ptr(), la.rank(),
                la.shape().data(), la.stride().data(), lb.stride().data(), node.dtype(), device.stream());
  return {out};
}

// ADD[a, b] (residual connections, gradient accumulation, a broadcast bias).
// runtime/__init__.mojo:319-333: contiguous operands take the flat kernel, views the strided one.
inline Buffers add(const OpRef& node, const Buffers& in, Device& device) {
  const Layout &la = node.src(0).layout(), &lb = node.src(1).layout();
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  if (detail::flat(node, in, 2))
    MOGRAD_CALL(device, mg_add, in[0].data_ptr(), in[1].data_ptr(), out.data_ptr(), node.numel(), node.dtype(),
                device.stream());
  else
    MOGRAD_CALL(device, mg_add_strided, in[0].data_ptr(), in[1].data_ptr(), out.data_ptr(), la.rank(), la.shape().data(),
                la.stride().data(), lb.stride().data(), node.dtype(), device.stream());
  return {out};
}

// RELU[a].  runtime/__init__.mojo:296-297.
inline Buffers relu(const OpRef& node, const Buffers& in, Device& device) {
  const Layout& l = node.src(0).layout();
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  if (detail::flat(node, in, 1))
    MOGRAD_CALL(device, mg_relu, in[0].data_ptr(), out.data_ptr(), node.numel(), node.dtype(), device.stream());
  else
    MOGRAD_CALL(device, mg_relu_strided, in[0].data_ptr(), out.data_ptr(), l.rank(), l.shape().data(), l.stride().data(),
                node.dtype(), device.stream());
  return {out};
}

// CAST[a] to node.dtype().  runtime/__init__.mojo:300-311.
inline Buffers cast(const OpRef& node, const Buffers& in, Device& device) {
  const Layout& l = node.src(0).layout();
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  if (detail::flat(node, in, 1))
    MOGRAD_CALL(device, mg_cast, in[0].data_ptr(), out.data_ptr(), node.numel(), node.src(0).dtype(), node.dtype(),
                device.stream());
  else
    MOGRAD_CALL(device, mg_cast_strided, in[0].data_ptr(), out.data_ptr(), l.rank(), l.shape().data(), l.stride().data(),
                node.src(0).dtype(), node.dtype(), device.stream());
  return {out};
}

// CONTIGUOUS[a]: row-major copy of a strided view.  runtime/__init__.mojo:456-461.
inline Buffers contiguous(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& l = node.src(0).layout();
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_contiguous, inputs[0].data_ptr(), out.data_ptr(), l.rank(), l.shape().data(), l.stride().data(),
              node.dtype(), device.stream());
  return {out};
}

// GATHER[src (rows, row_size), indices] -> (*indices.shape, row_size).
// runtime/__init__.mojo:239-240, kernels/__init__.mojo:132-163.
inline Buffers gather(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& la = node.src(0).layout();
  const Layout& lb = node.src(1).layout();
  if (la.rank() != 2) throw Error(MG_ERR_INVALID, "gather expects a 2D source tensor [num_rows, row_size]");  // op.mojo:367-368
  AnyBuffer idx = inputs[1];
  if (!lb.is_contiguous()) {  // strided indices: copy them row-major first
    idx = AnyBuffer::create(node.src(1).dtype(), device, lb.numel());
    MOGRAD_CALL(device, mg_contiguous, inputs[1].data_ptr(), idx.data_ptr(), lb.rank(), lb.shape().data(),
                lb.stride().data(), node.src(1).dtype(), device.stream());
  }
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_gather, inputs[0].data_ptr(), idx.data_ptr(), out.data_ptr(), lb.numel(), la.shape(0), la.shape(1),
              la.stride(0), la.stride(1), node.src(1).dtype(), node.dtype(), device.stream());
  return {out};
}

// SCATTER_ADD[indices, values (*indices.shape, row_size)] -> (num_rows, row_size).
// runtime/__init__.mojo:243-256; the output needs no zero fill here.
inline Buffers scatter_add(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& la = node.src(0).layout();
  const Layout& lb = node.src(1).layout();
  if (lb.rank() != la.rank() + 1)  // op.mojo:375-376
    throw Error(MG_ERR_INVALID, "scatter_add expects values shaped [*indices.shape, row_size]");
  const Buffers in = detail::materialise(node, inputs, device, 2);
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  if (device.pending)
    MOGRAD_CALL(device, mg_scatter_add_deferred, in[0].data_ptr(), in[1].data_ptr(), out.data_ptr(), la.numel(),
                node.shape(0), lb.shape(lb.rank() - 1), node.src(0).dtype(), node.dtype(), node.dtype(), device.pending,
                device.stream());
  else
    MOGRAD_CALL(device, mg_scatter_add, in[0].data_ptr(), in[1].data_ptr(), out.data_ptr(), la.numel(), node.shape(0),
                lb.shape(lb.rank() - 1), node.src(0).dtype(), node.dtype(), device.stream());
  return {out};
}

// SOFTMAX[a] over the last axis.  kernels/__init__.mojo:1015-1030.
inline Buffers softmax(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& l = node.src(0).layout();
  detail::require_float(node.dtype(), "softmax");
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  if (l.is_contiguous()) {
    const int64_t cols = l.shape(l.rank() - 1), rows = cols ? l.numel() / cols : 0;
    MOGRAD_CALL(device, mg_softmax, inputs[0].data_ptr(), out.data_ptr(), rows, cols, node.dtype(), device.stream());
  } else {  // kernels/__init__.mojo:1033-1060: views go to the strided kernel
    MOGRAD_CALL(device, mg_softmax_strided, inputs[0].data_ptr(), out.data_ptr(), l.rank(), l.shape().data(),
                l.stride().data(), node.dtype(), device.stream());
  }
  return {out};
}

// SOFTMAX_GRAD[y, upstream] (mograd/grad.mojo:232-234).  kernels/__init__.mojo:1062-1090.
inline Buffers softmax_grad(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& l = node.src(0).layout();
  const Buffers in = detail::materialise(node, inputs, device, 2);
  detail::require_float(node.dtype(), "softmax_grad");
  const int64_t size = l.shape(l.rank() - 1), N = l.numel() / size;
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_softmax_grad, in[0].data_ptr(), in[1].data_ptr(), out.data_ptr(), N, size, node.dtype(),
              device.stream());
  return {out};
}

// ARGMAX{axis}: index of the first largest value, stored in the tensor's float dtype.
// runtime/__init__.mojo:402-405; without `axis` the whole tensor is one lane.
inline Buffers argmax(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& l = node.src(0).layout();
  const Buffers in = detail::materialise(node, inputs, device, 1);
  detail::require_float(node.dtype(), "argmax");
  int64_t outer = 1, reduce = l.numel(), inner = 1;
  if (node.has_attr("axis")) l.reduce_dims(static_cast<int>(node.attr("axis")), outer, reduce, inner);
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_argmax_axis, in[0].data_ptr(), out.data_ptr(), outer, reduce, inner, node.dtype(), device.stream());
  return {out};
}

// ---- Exec functions of the fused nodes that the gradient rules below emit -----------------------------
// No counterpart in the reference: its Linear backward is matmul_grad + transpose_grad +
// expand_grad (mograd/grad.mojo:180-187,278-288), its LAYER_NORM has one output
// (mograd/runtime/__init__.mojo:425-426) and its labels are dense.  They follow the pattern of
// its multi-output FLASH_ATTN / FLASH_ATTN_GRAD pair (mograd/grad.mojo:309-344).

// LINEAR_GRAD[dY (.., N), X (.., K), W (N, K)(, prior)]{has_bias, relu_mask, accumulate} -> [dX, dW (N, K), db (N)]
// for Y = X W^T (+ b).  relu_mask: X is a ReLU's output and dX is zeroed where X <= 0; accumulate: dX = prior + dY W.
inline Buffers linear_bwd(const OpRef& node, const Buffers& in, Device& device) {
  const Layout &ldy = node.src(0).layout(), &lx = node.src(1).layout(), &lw = node.src(2).layout();
  const bool accumulate = node.has_attr("accumulate") && node.attr("accumulate") != 0;
  const bool relu_mask = node.has_attr("relu_mask") && node.attr("relu_mask") != 0;
  const Buffers inputs = detail::materialise(node, in, device, accumulate ? 4 : 3);
  detail::require_float(node.dtype(), "linear_bwd");
  if (lw.rank() != 2) throw Error(MG_ERR_INVALID, "linear_bwd: dY, X and W do not describe Y = X W^T");
  const int64_t N = lw.shape(0), K = lw.shape(1), M = lx.numel() / K;
  if (ldy.numel() != M * N) throw Error(MG_ERR_INVALID, "linear_bwd: dY, X and W do not describe Y = X W^T");
  const bool has_bias = !node.has_attr("has_bias") || node.attr("has_bias") != 0;
  AnyBuffer dx = AnyBuffer::create(node.dtype(), device, M * K);
  if (accumulate)  // the kernel adds into dx: start it from the prior gradient
    MOGRAD_CALL(device, mg_copy_device, dx.data_ptr(), inputs[3].data_ptr(), M * K * dtype_size(node.dtype()), device.stream());
  AnyBuffer dw = AnyBuffer::create(node.dtype(), device, N * K);
  Buffers out = {dx, dw};
  void* db_ptr = nullptr;
  if (has_bias) {
    out.push_back(AnyBuffer::create(node.dtype(), device, N));
    db_ptr = out.back().data_ptr();
  }
  if (device.pending)
    MOGRAD_CALL(device, mg_linear_bwd_deferred, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                dx.data_ptr(), dw.data_ptr(), db_ptr, M, N, K, accumulate, relu_mask, node.dtype(), node.dtype(),
                device.pending, device.stream());
  else if (accumulate || relu_mask)
    MOGRAD_CALL(device, mg_linear_bwd_fused, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), dx.data_ptr(),
                dw.data_ptr(), db_ptr, M, N, K, accumulate, relu_mask, node.dtype(), device.stream());
  else
    MOGRAD_CALL(device, mg_linear_bwd, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), dx.data_ptr(),
                dw.data_ptr(), db_ptr, M, N, K, node.dtype(), device.stream());
  return out;
}

// LAYER_NORM_STATS[x, gamma, beta]{eps} -> [y, mean (rows) f32, rstd (rows) f32].
inline Buffers layer_norm_fwd_stats(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& x = node.src(0).layout();
  const int64_t cols = x.shape(x.rank() - 1), rows = x.numel() / cols;
  detail::require_float(node.dtype(), "layer_norm_fwd_stats");
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  AnyBuffer mean = AnyBuffer::create(float32, device, rows);
  AnyBuffer rstd = AnyBuffer::create(float32, device, rows);
  MOGRAD_CALL(device, mg_layer_norm_fwd_stats, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
              out.data_ptr(), static_cast<float*>(mean.data_ptr()), static_cast<float*>(rstd.data_ptr()), rows, cols,
              static_cast<float>(node.attr("eps")),
              node.dtype(), device.stream());
  return {out, mean, rstd};
}

// LAYER_NORM_STATS_GRAD[dy, x, gamma, mean, rstd] -> [dx, dgamma, dbeta], and
// LAYER_NORM_STATS_GRAD_ADD[dy, x, gamma, mean, rstd, residual]: dx = gradient + residual.
inline Buffers layer_norm_bwd_stats(const OpRef& node, const Buffers& in, Device& device) {
  const Layout& x = node.src(1).layout();
  const Layout& gamma = node.src(2).layout();
  const int64_t cols = x.shape(x.rank() - 1), rows = x.numel() / cols;
  detail::require_float(node.dtype(), "layer_norm_bwd_stats");
  const bool with_residual = node.op_type == "LAYER_NORM_STATS_GRAD_ADD";
  const Buffers inputs = with_residual ? detail::materialise(node, in, device, 6) : in;
  AnyBuffer dx = AnyBuffer::create(node.dtype(), device, x.numel());
  AnyBuffer dgamma = AnyBuffer::create(node.dtype(), device, gamma.numel());
  AnyBuffer dbeta = AnyBuffer::create(node.dtype(), device, gamma.numel());
  const void* residual = with_residual ? inputs[5].data_ptr() : nullptr;
  const float* mean = static_cast<const float*>(inputs[3].data_ptr());
  const float* rstd = static_cast<const float*>(inputs[4].data_ptr());
  if (device.pending)
    MOGRAD_CALL(device, mg_layer_norm_bwd_stats_deferred, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                mean, rstd, residual, dx.data_ptr(), dgamma.data_ptr(), dbeta.data_ptr(), rows, cols, node.dtype(),
                node.dtype(), device.pending, device.stream());
  else if (with_residual)
    MOGRAD_CALL(device, mg_layer_norm_bwd_stats_add, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), mean,
                rstd, residual, dx.data_ptr(), dgamma.data_ptr(), dbeta.data_ptr(), rows, cols, node.dtype(),
                device.stream());
  else
    MOGRAD_CALL(device, mg_layer_norm_bwd_stats, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), mean,
                rstd, dx.data_ptr(), dgamma.data_ptr(), dbeta.data_ptr(), rows, cols, node.dtype(), device.stream());
  return {dx, dgamma, dbeta};
}

// LINEAR_LAYER_NORM_GRAD[dY (.., N), x (.., K), W (N, K), h (.., K), gamma, mean, rstd(, prior)]{has_bias, accumulate}
// -> [dh, dgamma, dbeta, dW, db] for Y = x W^T (+ b) with x = LayerNorm(h): the layer's LINEAR_GRAD and the
// LAYER_NORM_STATS_GRAD(_ADD) of the LayerNorm that feeds it as one node; dY W is never stored.
inline Buffers linear_layer_norm_bwd(const OpRef& node, const Buffers& in, Device& device) {
  const Layout &ldy = node.src(0).layout(), &lx = node.src(1).layout(), &lw = node.src(2).layout();
  const bool accumulate = node.has_attr("accumulate") && node.attr("accumulate") != 0;
  const bool has_bias = !node.has_attr("has_bias") || node.attr("has_bias") != 0;
  const Buffers inputs = detail::materialise(node, in, device, accumulate ? 8 : 7);
  detail::require_float(node.dtype(), "linear_layer_norm_bwd");
  if (lw.rank() != 2) throw Error(MG_ERR_INVALID, "linear_layer_norm_bwd: W is not a matrix");
  const int64_t N = lw.shape(0), K = lw.shape(1), M = lx.numel() / K;
  if (ldy.numel() != M * N || node.src(3).layout().numel() != M * K)
    throw Error(MG_ERR_INVALID, "linear_layer_norm_bwd: dY, x, W and h do not describe Y = LayerNorm(h) W^T");
  AnyBuffer dh = AnyBuffer::create(node.dtype(), device, M * K);
  if (accumulate)  // the kernel adds into dh: start it from the prior gradient
    MOGRAD_CALL(device, mg_copy_device, dh.data_ptr(), inputs[7].data_ptr(), M * K * dtype_size(node.dtype()), device.stream());
  AnyBuffer dgamma = AnyBuffer::create(node.dtype(), device, K);
  AnyBuffer dbeta = AnyBuffer::create(node.dtype(), device, K);
  AnyBuffer dw = AnyBuffer::create(node.dtype(), device, N * K);
  Buffers out = {dh, dgamma, dbeta, dw};
  void* db_ptr = nullptr;
  if (has_bias) {
    out.push_back(AnyBuffer::create(node.dtype(), device, N));
    db_ptr = out.back().data_ptr();
  }
  MOGRAD_CALL(device, mg_linear_bwd_layer_norm_bwd, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
              inputs[3].data_ptr(), inputs[4].data_ptr(), static_cast<const float*>(inputs[5].data_ptr()),
              static_cast<const float*>(inputs[6].data_ptr()), dh.data_ptr(), dw.data_ptr(), db_ptr, dgamma.data_ptr(),
              dbeta.data_ptr(), M, N, K, accumulate, node.dtype(), node.dtype(), device.pending, device.stream());
  return out;
}

// MATMUL_BT_ADD[A, B (N, K), R] = A B^T + R, R laid out like the result.
inline Buffers matmul_bt_add(const OpRef& node, const Buffers& inputs, Device& device) {
  const int64_t N = node.shape(node.layout().rank() - 1);
  const detail::MatmulDims d = detail::matmul_dims(node.src(0).layout(), node.src(1).layout(), N, true, "matmul");
  AnyBuffer residual = inputs[2];
  if (!node.src(2).layout().is_contiguous()) {
    const OpRef wrap{"ADD", node.layout(), node.dtype(), {node.src(2)}, {}};
    residual = detail::materialise(wrap, {inputs[2]}, device, 1)[0];
  }
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_matmul_bt_add, inputs[0].data_ptr(), inputs[1].data_ptr(), residual.data_ptr(), out.data_ptr(),
              d.batch, d.M, N, d.K, d.lda0, d.lda1, d.ldb0, d.ldb1, d.bsa, d.bsb, node.dtype(), device.stream());
  return {out};
}

// MATMUL_BIAS_RELU_BT[A, B (N, K), bias (N)] = max(A B^T + bias, 0).
inline Buffers matmul_bias_relu_bt(const OpRef& node, const Buffers& inputs, Device& device) {
  const int64_t N = node.shape(node.layout().rank() - 1);
  const detail::MatmulDims d = detail::matmul_dims(node.src(0).layout(), node.src(1).layout(), N, true, "matmul_bias");
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_matmul_bias_relu_bt, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
              out.data_ptr(), d.batch, d.M, N, d.K, d.lda0, d.lda1, d.ldb0, d.ldb1, d.bsa, d.bsb, node.dtype(),
              device.stream());
  return {out};
}

// RESHAPE[a]: a contiguous tensor under another shape, a view (a strided source is materialised first).
inline Buffers reshape(const OpRef& node, const Buffers& inputs, Device& device) {
  const Buffers in = detail::materialise(node, inputs, device, 1);
  const Layout rows = node.layout().as_contiguous();
  return {in[0].view(Layout(rows.shape(), rows.stride(), in[0].offset_elems()))};
}

// TRANSPOSE[a]{dim0, dim1}: a strided view of the same storage.
inline Buffers transpose(const OpRef& node, const Buffers& inputs, Device&) { return {inputs[0].view(node.layout())}; }
// EXPAND[a]: a broadcast view, stride 0 along the expanded axes (what grad.mojo:156-177 builds as
// the gradient of SUM); consumers materialise it with mg_contiguous.
inline Buffers expand(const OpRef& node, const Buffers& inputs, Device&) { return {inputs[0].view(node.layout())}; }

// FLASH_ATTN_PACKED[qkv (B, S, 3, H, D)(, mask)]{scale, is_causal, has_bias} -> [O (B, S, H, D), LSE (B, H, S) f32].
inline Buffers flash_attn_packed_fwd(const OpRef& node, const Buffers& inputs, Device& device) {
  const Layout& q = node.src(0).layout();
  if (q.rank() != 5 || q.shape(2) != 3) throw Error(MG_ERR_INVALID, "flash_attn_packed: qkv must be (B, S, 3, H, D)");
  const int64_t B = q.shape(0), S = q.shape(1), H = q.shape(3), D = q.shape(4);
  const bool is_causal = node.attr("is_causal") != 0;
  const bool has_bias = node.has_attr("has_bias") ? node.attr("has_bias") != 0 : true;
  detail::require_float(node.dtype(), "flash_attn_fwd");
  AnyBuffer dst = AnyBuffer::create(node.dtype(), device, node.numel());
  AnyBuffer lse = AnyBuffer::create(float32, device, B * H * S);
  const void* mask = inputs.size() > 1 ? inputs[1].data_ptr() : nullptr;
  MOGRAD_CALL(device, mg_flash_attn_fwd_packed, inputs[0].data_ptr(), mask, dst.data_ptr(),
              static_cast<float*>(lse.data_ptr()), B, S, H, D, static_cast<float>(node.attr("scale")), is_causal, has_bias,
              node.dtype(), device.stream());
  return {dst, lse};
}

// FLASH_ATTN_PACKED_GRAD[dO, O, qkv, LSE(, mask)] -> dqkv (B, S, 3, H, D).
inline Buffers flash_attn_packed_bwd(const OpRef& node, const Buffers& in, Device& device) {
  const Layout& q = node.src(2).layout();
  const int64_t B = q.shape(0), S = q.shape(1), H = q.shape(3), D = q.shape(4);
  const bool is_causal = node.attr("is_causal") != 0;
  const bool has_bias = node.has_attr("has_bias") ? node.attr("has_bias") != 0 : !is_causal;
  detail::require_float(node.dtype(), "flash_attn_bwd");
  const Buffers inputs = detail::materialise(node, in, device, 1);
  AnyBuffer dqkv = AnyBuffer::create(node.dtype(), device, node.numel());
  const void* mask = inputs.size() > 4 ? inputs[4].data_ptr() : nullptr;
  MOGRAD_CALL(device, mg_flash_attn_bwd_packed, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), mask,
              static_cast<const float*>(inputs[3].data_ptr()), dqkv.data_ptr(), B, S, H, D,
              static_cast<float>(node.attr("scale")), is_causal, has_bias, node.dtype(), device.stream());
  return {dqkv};
}

// CROSS_ENTROPY_IDS[logits (.., C), ids (..) int32/int64] -> (1,).
inline Buffers cross_entropy_ids(const OpRef& node, const Buffers& in, Device& device) {
  const Layout& la = node.src(0).layout();
  const Buffers inputs = detail::materialise(node, in, device, 2);
  detail::require_float(node.dtype(), "cross_entropy_ids");
  const int64_t C = la.shape(la.rank() - 1), N = la.numel() / C;
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_cross_entropy_ids, inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), N, C, node.dtype(),
              node.src(1).dtype(), device.stream());
  return {out};
}

// CROSS_ENTROPY_IDS_GRAD[logits, ids, upstream (1,)] -> dlogits.
inline Buffers cross_entropy_grad_ids(const OpRef& node, const Buffers& in, Device& device) {
  const Layout& la = node.src(0).layout();
  const Buffers inputs = detail::materialise(node, in, device, 2);
  detail::require_float(node.dtype(), "cross_entropy_grad_ids");
  const int64_t C = la.shape(la.rank() - 1), N = la.numel() / C;
  AnyBuffer out = AnyBuffer::create(node.dtype(), device, node.numel());
  MOGRAD_CALL(device, mg_cross_entropy_grad_ids, inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
              out.data_ptr(), N, C, node.dtype(), node.src(1).dtype(), device.stream());
  return {out};
}

// ---- Gradient rules (GradFn, mograd/grad.mojo:12): node + upstream -> the multi-output node that
// computes every source's gradient.  The C++ side keeps the rules that the reference lacks
// (mograd/grad.mojo:30-65 has none for MATMUL_BT / MATMUL_BIAS_BT); output i of the returned node is
// the gradient of source i, which the caller selects as the reference selects with GETTUPLE. ----------

// MATMUL_BIAS_BT[X, W, b] or MATMUL_BT[X, W], upstream dY -> LINEAR_GRAD[dY, X, W]{has_bias}.
inline OpRef linear_grad(const OpRef& node, const OpRef& upstream) {
  const bool has_bias = node.op_type == "MATMUL_BIAS_BT";
  return OpRef{"LINEAR_GRAD", node.src(0).layout().as_contiguous(), node.src(0).dtype(),
               {upstream, node.src(0), node.src(1)}, {{"has_bias", has_bias ? 1.0 : 0.0}}};
}

// LAYER_NORM_STATS[x, gamma, beta] with its outputs 1 and 2 (mean, rstd) given as leaves ->
// LAYER_NORM_STATS_GRAD[dy, x, gamma, mean, rstd].
inline OpRef layer_norm_stats_grad(const OpRef& node, const OpRef& upstream, const OpRef& mean, const OpRef& rstd) {
  return OpRef{"LAYER_NORM_STATS_GRAD", node.src(0).layout().as_contiguous(), node.src(0).dtype(),
               {upstream, node.src(0), node.src(1), mean, rstd}, {}};
}

// CROSS_ENTROPY_IDS[logits, ids], upstream (1,) -> CROSS_ENTROPY_IDS_GRAD[logits, ids, upstream].
inline OpRef cross_entropy_ids_grad(const OpRef& node, const OpRef& upstream) {
  return OpRef{"CROSS_ENTROPY_IDS_GRAD", node.src(0).layout().as_contiguous(), node.src(0).dtype(),
               {node.src(0), node.src(1), upstream}, {}};
}

// ---- Rewrite rules (RewriteFn, mograd/simplify/__init__.mojo:9): node -> the fused node, or nothing.  The
// fusions of a transformer training step that this library adds to the reference's GPU_REWRITES
// (mograd/runtime/gpu/rewrites.mojo:13-34).  A multi-output node's result i is selected by
// GETTUPLE{index: i}[node], as in the reference. -------------------------------------------------------------

inline OpRef gettuple(const OpRef& src, int index, const Layout& layout, DType dtype) {
  return OpRef{"GETTUPLE", layout, dtype, {src}, {{"index", static_cast<double>(index)}}};
}
inline bool is_output0_of(const OpRef& n, const char* op) {
  return n.op_type == "GETTUPLE" && n.attr("index") == 0 && n.src(0).op_type == op;
}

// ADD(MATMUL_BT(a, w), r), either operand order -> MATMUL_BT_ADD[a, w, r].
inline std::optional<OpRef> fuse_matmul_add(const OpRef& node) {
  if (node.op_type != "ADD") return std::nullopt;
  for (int i = 0; i < 2; ++i) {
    const OpRef &mm = node.src(i), &other = node.src(1 - i);
    if (mm.op_type == "MATMUL_BT" && mm.layout().shape() == other.layout().shape() && mm.dtype() == other.dtype())
      return OpRef{"MATMUL_BT_ADD", mm.layout(), node.dtype(), {mm.src(0), mm.src(1), other}, {}};
  }
  return std::nullopt;
}

// RELU(MATMUL_BIAS_BT(a, w, b)) -> MATMUL_BIAS_RELU_BT[a, w, b].
inline std::optional<OpRef> fuse_matmul_bias_relu(const OpRef& node) {
  if (node.op_type != "RELU" || node.src(0).op_type != "MATMUL_BIAS_BT") return std::nullopt;
  return OpRef{"MATMUL_BIAS_RELU_BT", node.src(0).layout(), node.dtype(), node.src(0).srcs, {}};
}

// RELU_GRAD(y, GETTUPLE0(LINEAR_GRAD(dy, y, w))) -> GETTUPLE0(LINEAR_GRAD{relu_mask}(dy, y, w)); `same` tells
// whether two operand positions hold the same tensor (nodes here are values, not graph vertices).
inline std::optional<OpRef> fuse_relu_grad_into_linear_grad(const OpRef& node, bool x_is_the_relu_output) {
  if (node.op_type != "RELU_GRAD" || !is_output0_of(node.src(1), "LINEAR_GRAD") || !x_is_the_relu_output) return std::nullopt;
  OpRef lin = node.src(1).src(0);
  if (lin.has_attr("relu_mask") || lin.has_attr("accumulate")) return std::nullopt;
  lin.node_attrs["relu_mask"] = 1.0;
  return gettuple(lin, 0, node.src(1).layout(), node.src(1).dtype());
}

// ADD(p, GETTUPLE0(LINEAR_GRAD(dy, x, w))) -> GETTUPLE0(LINEAR_GRAD{accumulate}(dy, x, w, p)).
inline std::optional<OpRef> fuse_add_into_linear_grad(const OpRef& node) {
  if (node.op_type != "ADD") return std::nullopt;
  for (int i = 0; i < 2; ++i) {
    const OpRef &sel = node.src(i), &other = node.src(1 - i);
    if (!is_output0_of(sel, "LINEAR_GRAD") || sel.src(0).has_attr("accumulate")) continue;
    if (sel.layout().shape() != other.layout().shape() || sel.dtype() != other.dtype()) continue;
    OpRef lin = sel.src(0);
    lin.srcs.push_back(other);
    lin.node_attrs["accumulate"] = 1.0;
    return gettuple(lin, 0, sel.layout(), sel.dtype());
  }
  return std::nullopt;
}

// ADD(r, GETTUPLE0(LAYER_NORM_STATS_GRAD(dy, x, g, mean, rstd))) -> GETTUPLE0(LAYER_NORM_STATS_GRAD_ADD(.., r)).
inline std::optional<OpRef> fuse_add_into_layer_norm_grad(const OpRef& node) {
  if (node.op_type != "ADD") return std::nullopt;
  for (int i = 0; i < 2; ++i) {
    const OpRef &sel = node.src(i), &other = node.src(1 - i);
    if (!is_output0_of(sel, "LAYER_NORM_STATS_GRAD")) continue;
    if (sel.layout().shape() != other.layout().shape() || sel.dtype() != other.dtype()) continue;
    OpRef ln = sel.src(0);
    ln.op_type = "LAYER_NORM_STATS_GRAD_ADD";
    ln.srcs.push_back(other);
    return gettuple(ln, 0, sel.layout(), sel.dtype());
  }
  return std::nullopt;
}

// LAYER_NORM_STATS_GRAD(_ADD)(GETTUPLE0(LINEAR_GRAD(dy, x, w)), h, g, mean, rstd(, r)) ->
// LINEAR_LAYER_NORM_GRAD[dy, x, w, h, g, mean, rstd(, r)]: outputs [dh, dgamma, dbeta, dW, db], so the selectors
// of the LayerNorm node keep their indices and the product's dW and db are read at 3 and 4.  The caller
// applies it only where nothing else reads the product's dX.
inline std::optional<OpRef> fuse_linear_grad_into_layer_norm_grad(const OpRef& node) {
  const bool with_residual = node.op_type == "LAYER_NORM_STATS_GRAD_ADD";
  if ((node.op_type != "LAYER_NORM_STATS_GRAD" && !with_residual) || !is_output0_of(node.src(0), "LINEAR_GRAD"))
    return std::nullopt;
  const OpRef& lin = node.src(0).src(0);
  if (lin.has_attr("relu_mask") || lin.has_attr("accumulate") || lin.dtype() != node.dtype()) return std::nullopt;
  if (node.src(1).layout().numel() != node.src(0).layout().numel()) return std::nullopt;
  OpRef fused{"LINEAR_LAYER_NORM_GRAD", node.layout(), node.dtype(),
              {lin.src(0), lin.src(1), lin.src(2), node.src(1), node.src(2), node.src(3), node.src(4)},
              {{"has_bias", !lin.has_attr("has_bias") || lin.attr("has_bias") != 0 ? 1.0 : 0.0}}};
  if (with_residual) {
    fused.srcs.push_back(node.src(5));
    fused.node_attrs["accumulate"] = 1.0;
  }
  return fused;
}

// ADD(r, GETTUPLE0(LINEAR_LAYER_NORM_GRAD(..))) -> GETTUPLE0(LINEAR_LAYER_NORM_GRAD{accumulate}(.., r)).
inline std::optional<OpRef> fuse_add_into_linear_layer_norm_grad(const OpRef& node) {
  if (node.op_type != "ADD") return std::nullopt;
  for (int i = 0; i < 2; ++i) {
    const OpRef &sel = node.src(i), &other = node.src(1 - i);
    if (!is_output0_of(sel, "LINEAR_LAYER_NORM_GRAD") || sel.src(0).has_attr("accumulate")) continue;
    if (sel.layout().shape() != other.layout().shape() || sel.dtype() != other.dtype()) continue;
    OpRef fused = sel.src(0);
    fused.srcs.push_back(other);
    fused.node_attrs["accumulate"] = 1.0;
    return gettuple(fused, 0, sel.layout(), sel.dtype());
  }
  return std::nullopt;
}

// CONTIGUOUS(TRANSPOSE{1,2}(GETTUPLE0(FLASH_ATTN(q, k, v, mask)))) -> GETTUPLE0(FLASH_ATTN{layout: bshd}(...)).
inline std::optional<OpRef> fuse_attention_output_layout(const OpRef& node) {
  if (node.op_type != "CONTIGUOUS" || node.src(0).op_type != "TRANSPOSE" || !is_output0_of(node.src(0).src(0), "FLASH_ATTN"))
    return std::nullopt;
  const OpRef& tr = node.src(0);
  const OpRef& sel = tr.src(0);
  const int d0 = (static_cast<int>(tr.has_attr("dim0") ? tr.attr("dim0") : -2) + 4) % 4;
  const int d1 = (static_cast<int>(tr.has_attr("dim1") ? tr.attr("dim1") : -1) + 4) % 4;
  if (tr.layout().rank() != 4 || !((d0 == 1 && d1 == 2) || (d0 == 2 && d1 == 1))) return std::nullopt;
  OpRef attn = sel.src(0);
  if (attn.has_attr("layout")) return std::nullopt;
  attn.node_attrs["layout"] = kLayoutBshd;
  const Layout bshd({sel.shape(0), sel.shape(2), sel.shape(1), sel.shape(3)});
  attn.node_layout = bshd;
  return gettuple(attn, 0, bshd, sel.dtype());
}

// Leaves the second-stage sums of the exec functions that run inside its lifetime on one mg_deferred list
// and finishes them with a single launch (finish()), as a training step does at its end.
class DeferredSums {
 public:
  explicit DeferredSums(Device& device) : device_(device) {
    MOGRAD_CALL(device_, mg_deferred_create, &device_.pending);
  }
  ~DeferredSums() {
    if (device_.pending) device_.fn<decltype(&::mg_deferred_destroy)>("mg_deferred_destroy")(device_.pending);
    device_.pending = nullptr;
  }
  void finish() { MOGRAD_CALL(device_, mg_finish_deferred, device_.pending, device_.stream()); }

 private:
  Device& device_;
};

// ---- Rule table (mograd/runtime/__init__.mojo:113-167) --------------------------------------------------

struct Rule {
  const char* op_type;
  const char* exec_name;
  BoundExecFn fn;
};

// The rows of the reference's rule table that belong to this path, in its order.
inline const std::vector<Rule>& scheduler_rules() {
  static const std::vector<Rule> rules = {
      {"ADD", "add", add},
      {"RELU", "relu", relu},
      {"CAST", "cast", cast},
      {"CONTIGUOUS", "contiguous", contiguous},
      {"GATHER", "gather", gather},
      {"SCATTER_ADD", "scatter_add", scatter_add},
      {"RELU_GRAD", "relu_grad", relu_grad},
      {"SOFTMAX", "softmax", softmax},
      {"SOFTMAX_GRAD", "softmax_grad", softmax_grad},
      {"ARGMAX", "argmax", argmax},
      {"SUM", "sum", sum},
      {"MATMUL", "matmul", matmul},
      {"MATMUL_BT", "matmul_t", matmul_t},
      {"MATMUL_BIAS_BT", "matmul_bias_bt", matmul_bias_bt},
      {"LAYER_NORM", "layer_norm_fwd", layer_norm_fwd},
      {"LAYER_NORM_GRAD", "layer_norm_bwd", layer_norm_bwd},
      {"FLASH_ATTN", "flash_attn_fwd_sched", flash_attn_fwd_sched},
      {"FLASH_ATTN_GRAD", "flash_attn_bwd_sched", flash_attn_bwd_sched},
      {"CROSS_ENTROPY", "cross_entropy", cross_entropy},
      {"CROSS_ENTROPY_GRAD", "cross_entropy_grad", cross_entropy_grad},
      // fused nodes emitted by the gradient rules above (no counterpart in the reference's table)
      {"LINEAR_GRAD", "linear_bwd", linear_bwd},
      {"LAYER_NORM_STATS", "layer_norm_fwd_stats", layer_norm_fwd_stats},
      {"LAYER_NORM_STATS_GRAD", "layer_norm_bwd_stats", layer_norm_bwd_stats},
      {"CROSS_ENTROPY_IDS", "cross_entropy_ids", cross_entropy_ids},
      {"CROSS_ENTROPY_IDS_GRAD", "cross_entropy_grad_ids", cross_entropy_grad_ids},
      // views, and the fused nodes that the rewrite rules below create
      {"RESHAPE", "reshape", reshape},
      {"TRANSPOSE", "transpose", transpose},
      {"EXPAND", "expand", expand},
      {"MATMUL_BT_ADD", "matmul_bt_add", matmul_bt_add},
      {"MATMUL_BIAS_RELU_BT", "matmul_bias_relu_bt", matmul_bias_relu_bt},
      {"LAYER_NORM_STATS_GRAD_ADD", "layer_norm_bwd_stats", layer_norm_bwd_stats},
      {"LINEAR_LAYER_NORM_GRAD", "linear_layer_norm_bwd", linear_layer_norm_bwd},
      {"FLASH_ATTN_PACKED", "flash_attn_packed_fwd", flash_attn_packed_fwd},
      {"FLASH_ATTN_PACKED_GRAD", "flash_attn_packed_bwd", flash_attn_packed_bwd},
  };
  return rules;
}

// One scheduler step: the first matching rule wins (pattern_matcher.mojo:74-80).
inline Buffers run(const OpRef& node, const Buffers& inputs, Device& device) {
  for (const Rule& r : scheduler_rules())
    if (node.op_type == r.op_type) return r.fn(node, inputs, device);
  throw Error(MG_ERR_UNSUPPORTED, "no scheduler rule for op " + node.op_type + " on the backward hot path");
}

}  // namespace mograd
