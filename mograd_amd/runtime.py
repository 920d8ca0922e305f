"""Host-side mirror of mograd's kernel-dispatch surface for the backward hot path.

The reference's scheduler maps an op node to a `BoundExecFn(node, inputs, device) ->
List[AnyBuffer]` (mograd/scheduler.mojo:13-15) whose body marshals layouts into a
kernel call (mograd/runtime/gpu/kernels/dispatch.mojo).  This module restates that
surface in Python over libmograd_hip.so, with the same names, argument derivations
and error conditions, so that tests of the HIP kernels read like the reference's own
tests.  It contains no arithmetic: every result comes from the C ABI.

    Layout      shape + element strides + base offset      mograd/layout.mojo:15-28
    Device      stream + pool handle                       mograd/device_ctx.mojo:25-113
    AnyBuffer   typed device allocation from the pool      mograd/buffer.mojo:135-214
    Node        (op_type, layout, dtype, srcs, attrs)      mograd/op.mojo:124-185
    SCHEDULER_RULES   op type -> exec function             mograd/runtime/__init__.mojo:113-167
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import _lib
from ._lib import BF16, F16, F32, I32, I64, MogradError

__all__ = [
    "Layout", "Device", "AnyBuffer", "Node", "SCHEDULER_RULES", "GRAD_RULES", "gradient", "evaluate", "MogradError",
    "float32", "float16", "bfloat16", "int32", "int64",
]

float32, float16, bfloat16, int32, int64 = F32, F16, BF16, I32, I64

_NP_OF = {F32: np.float32, F16: np.float16, I32: np.int32, I64: np.int64}


# --------------------------------------------------------------------------- #
# bfloat16 <-> float32 on the host (numpy has no bfloat16)
# --------------------------------------------------------------------------- #


def f32_to_bf16_bits(a) -> np.ndarray:
    """Round-to-nearest-even float32 -> bfloat16 bit patterns (uint16)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(bits) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_to_dtype(a, dtype: int) -> np.ndarray:
    """`a` rounded once to `dtype`, returned as float32 (what the kernel will see)."""
    a = np.asarray(a, dtype=np.float32)
    if dtype == F32:
        return a
    if dtype == F16:
        return a.astype(np.float16).astype(np.float32)
    if dtype == BF16:
        return bf16_bits_to_f32(f32_to_bf16_bits(a)).reshape(a.shape)
    raise ValueError(f"not a float dtype: {dtype}")


# --------------------------------------------------------------------------- #
# Layout
# --------------------------------------------------------------------------- #


def _row_major(shape: Sequence[int]) -> Tuple[int, ...]:
    strides = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        strides[i] = strides[i + 1] * shape[i + 1]
    return tuple(strides)


@dataclass(frozen=True)
class Layout:
    """Shape, element strides and base offset (mograd/layout.mojo)."""

    dims: Tuple[int, ...]
    strides: Tuple[int, ...] = ()
    base_offset: int = 0

    def __init__(self, *shape, strides: Optional[Sequence[int]] = None, base_offset: int = 0):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        object.__setattr__(self, "dims", tuple(int(s) for s in shape))
        st = _row_major(self.dims) if strides is None else tuple(int(s) for s in strides)
        if len(st) != len(self.dims):
            raise ValueError("strides rank differs from shape rank")
        object.__setattr__(self, "strides", st)
        object.__setattr__(self, "base_offset", int(base_offset))

    def rank(self) -> int:
        return len(self.dims)

    def shape(self, idx: Optional[int] = None):
        return self.dims if idx is None else self.dims[idx]

    def stride(self, idx: Optional[int] = None):
        return self.strides if idx is None else self.strides[idx]

    def numel(self) -> int:
        n = 1
        for s in self.dims:
            n *= s
        return n

    def is_contiguous(self) -> bool:  # layout.mojo:210-212
        return self.strides == _row_major(self.dims)

    def as_contiguous(self) -> "Layout":  # layout.mojo:238-240
        return Layout(*self.dims)

    def batch_dims_collapsible(self) -> bool:  # layout.mojo:214-236
        for i in range(self.rank() - 4, -1, -1):
            if self.strides[i] != self.dims[i + 1] * self.strides[i + 1]:
                return False
        return True

    def reduce_dims(self, axis: int) -> Tuple[int, int, int]:  # layout.mojo:287-298
        ax = axis + self.rank() if axis < 0 else axis
        if not 0 <= ax < self.rank():
            raise MogradError(1, f"axis {axis} out of range for rank {self.rank()}")
        reduce_size = self.dims[ax]
        inner = 1
        for s in self.dims[ax + 1:]:
            inner *= s
        outer = self.numel() // (reduce_size * inner)
        return outer, reduce_size, inner

    def transpose(self, dim0: int = -2, dim1: int = -1) -> "Layout":  # layout.mojo:435-452
        d0 = dim0 % self.rank()
        d1 = dim1 % self.rank()
        dims = list(self.dims)
        st = list(self.strides)
        dims[d0], dims[d1] = dims[d1], dims[d0]
        st[d0], st[d1] = st[d1], st[d0]
        return Layout(*dims, strides=st, base_offset=self.base_offset)

    def slice_axis(self, axis: int, start: int, stop: int, step: int = 1) -> "Layout":  # layout.mojo:321-340
        ax = axis % self.rank()
        extent = max(0, (stop - start + step - 1) // step)
        dims = list(self.dims)
        st = list(self.strides)
        dims[ax] = extent
        st[ax] = self.strides[ax] * step
        return Layout(*dims, strides=st, base_offset=self.base_offset + start * self.strides[ax])


# --------------------------------------------------------------------------- #
# Device and buffers
# --------------------------------------------------------------------------- #


class Device:
    """One GPU, one in-order stream, and the process-wide caching pool
    (mograd/device_ctx.mojo:25-113).  Raises if the HIP library is missing."""

    def __init__(self, index: int = 0):
        self.lib = _lib.load()
        self.lib.mg_init(index)
        self.index = index
        s = C.c_void_p()
        self.lib.mg_stream_create(C.byref(s))
        self.stream = s

    def synchronize(self) -> None:
        self.lib.mg_stream_sync(self.stream)

    # The list on which the exec functions of LINEAR_GRAD, LAYER_NORM_STATS_GRAD(_ADD) and
    # SCATTER_ADD leave their second-stage sums while it is set (see `deferred_sums`).
    pending = None

    def empty_cache(self) -> None:
        self.lib.mg_pool_empty_cache()

    def memory_stats(self) -> _lib.PoolStats:
        st = _lib.PoolStats()
        self.lib.mg_pool_get_stats(C.byref(st))
        return st

    def memory_summary(self) -> str:
        n = self.lib.mg_pool_summary(None, 0)
        buf = C.create_string_buffer(int(n) + 1)
        self.lib.mg_pool_summary(buf, n + 1)
        return buf.value.decode()

    def pool_enabled(self) -> bool:
        return bool(self.lib.mg_pool_enabled())

    def cu_count(self) -> int:
        return int(self.lib.mg_device_cu_count())

    def close(self) -> None:
        if self.stream is not None:
            self.lib.mg_stream_sync(self.stream)
            self.lib.mg_stream_destroy(self.stream)
            self.stream = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class _Storage:
    """One pooled allocation; returns to the free lists when the last view dies
    (Storage, mograd/memory.mojo:199-239)."""

    def __init__(self, device: Device, nbytes: int):
        self.device = device
        self.lib = device.lib
        p = C.c_void_p()
        self.lib.mg_pool_alloc(C.byref(p), nbytes)
        self.ptr = p.value or 0
        self.nbytes = nbytes

    def __del__(self):
        try:
            if self.ptr:
                self.lib.mg_pool_free(C.c_void_p(self.ptr))
                self.ptr = 0
        except Exception:
            pass


class AnyBuffer:
    """A typed device buffer (mograd/buffer.mojo:135-214).  `view` shares storage."""

    def __init__(self, storage: _Storage, dtype: int, numel: int, offset_elems: int = 0):
        self.storage = storage
        self.dtype = dtype
        self.numel = numel
        self.offset_elems = offset_elems

    @staticmethod
    def supports(dtype: int) -> bool:
        return dtype in _lib.DTYPE_SIZE

    @staticmethod
    def create(dtype: int, device: Device, numel: int, fill: Optional[float] = None) -> "AnyBuffer":
        if dtype not in _lib.DTYPE_SIZE:
            raise MogradError(1, f"Unsupported dtype: {dtype}")
        buf = AnyBuffer(_Storage(device, numel * _lib.DTYPE_SIZE[dtype]), dtype, numel)
        if fill is not None:
            device.lib.mg_fill(buf.data_ptr(), float(fill), numel, dtype, device.stream)
        return buf

    @staticmethod
    def from_numpy(device: Device, array, dtype: Optional[int] = None) -> "AnyBuffer":
        """Uploads `array`.  Float arrays are rounded once to `dtype` (default float32)."""
        a = np.asarray(array)
        if dtype is None:
            dtype = {np.dtype(np.int32): I32, np.dtype(np.int64): I64, np.dtype(np.float16): F16}.get(a.dtype, F32)
        if dtype == BF16:
            host = f32_to_bf16_bits(a.astype(np.float32)).reshape(-1)
        else:
            host = np.ascontiguousarray(a, dtype=_NP_OF[dtype]).reshape(-1)
        buf = AnyBuffer.create(dtype, device, host.size)
        device.lib.mg_copy_to_device(buf.data_ptr(), host.ctypes.data_as(C.c_void_p), host.nbytes, device.stream)
        return buf

    def data_ptr(self, with_offset: bool = True) -> C.c_void_p:
        off = self.offset_elems * _lib.DTYPE_SIZE[self.dtype] if with_offset else 0
        return C.c_void_p(self.storage.ptr + off)

    def size_bytes(self) -> int:
        return self.numel * _lib.DTYPE_SIZE[self.dtype]

    def view(self, layout: Layout) -> "AnyBuffer":
        return AnyBuffer(self.storage, self.dtype, layout.numel(), layout.base_offset)

    def to_numpy(self, shape: Optional[Sequence[int]] = None) -> np.ndarray:
        """Synchronous download.  bfloat16 comes back as float32."""
        dev = self.storage.device
        if self.dtype == BF16:
            host = np.empty(self.numel, dtype=np.uint16)
        else:
            host = np.empty(self.numel, dtype=_NP_OF[self.dtype])
        dev.lib.mg_copy_to_host(host.ctypes.data_as(C.c_void_p), self.data_ptr(), host.nbytes, dev.stream)
        out = bf16_bits_to_f32(host) if self.dtype == BF16 else host
        return out.reshape(tuple(shape)) if shape is not None else out

    def item(self) -> float:
        return self.to_numpy().reshape(-1)[0].item()


# --------------------------------------------------------------------------- #
# Op nodes
# --------------------------------------------------------------------------- #


@dataclass(eq=False)
class Node:
    """Just enough of an op node for the exec functions: its own layout and dtype, the
    layouts of its sources, and its attributes (mograd/op.mojo:124-185)."""

    op_type: str
    node_layout: Layout
    node_dtype: int
    srcs: List["Node"] = field(default_factory=list)
    node_attrs: Dict[str, object] = field(default_factory=dict)
    # What the reference keeps in op().buf (mograd/scheduler.mojo:74-78): a leaf's buffer, or
    # the cached results of an evaluated node (several for a multi-output node).
    bufs: Optional[List["AnyBuffer"]] = field(default=None, repr=False, compare=False)

    def layout(self) -> Layout:
        return self.node_layout

    def dtype(self) -> int:
        return self.node_dtype

    def numel(self) -> int:
        return self.node_layout.numel()

    def src(self, i: int) -> "Node":
        return self.srcs[i]

    def attrs(self) -> Dict[str, object]:
        return self.node_attrs

    def shape(self, i: int) -> int:
        return self.node_layout.shape(i)

    @staticmethod
    def leaf(layout: Layout, dtype: int = F32, buf: Optional["AnyBuffer"] = None) -> "Node":
        return Node("BUFFER", layout, dtype, bufs=None if buf is None else [buf])

    def __hash__(self) -> int:  # nodes are graph vertices: identity, like OpRef
        return id(self)

    def __eq__(self, other) -> bool:
        return self is other


def _require_float(dtype: int, who: str) -> None:
    if dtype not in (F32, F16, BF16):  # dispatch_dtype[float_only=True], dispatch.mojo:564-576
        raise MogradError(1, f"{who}: unsupported dtype")


# --------------------------------------------------------------------------- #
# Exec functions (BoundExecFn bodies)
# --------------------------------------------------------------------------- #


def layer_norm_fwd(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """LAYER_NORM[x, gamma, beta]{eps}.  dispatch.mojo:294-314."""
    x_layout = node.src(0).layout()
    cols = x_layout.shape(x_layout.rank() - 1)
    rows = x_layout.numel() // cols
    eps = float(node.attrs()["eps"])
    _require_float(node.dtype(), "layer_norm_fwd")
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_layer_norm_fwd(inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), out.data_ptr(),
                                 rows, cols, eps, node.dtype(), device.stream)
    return [out]


def layer_norm_bwd(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """LAYER_NORM_GRAD[dy, x, gamma]{eps} -> [dx, dgamma, dbeta].  dispatch.mojo:332-358."""
    x_layout = node.src(1).layout()
    gamma_layout = node.src(2).layout()
    cols = x_layout.shape(x_layout.rank() - 1)
    rows = x_layout.numel() // cols
    eps = float(node.attrs()["eps"])
    _require_float(node.dtype(), "layer_norm_bwd")
    dx = AnyBuffer.create(node.dtype(), device, x_layout.numel())
    dgamma = AnyBuffer.create(node.dtype(), device, gamma_layout.numel())
    dbeta = AnyBuffer.create(node.dtype(), device, gamma_layout.numel())
    device.lib.mg_layer_norm_bwd(inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), dx.data_ptr(),
                                 dgamma.data_ptr(), dbeta.data_ptr(), rows, cols, eps, node.dtype(), device.stream)
    return [dx, dgamma, dbeta]


def flash_attn_fwd_sched(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """FLASH_ATTN[Q, K, V, mask]{scale, is_causal, has_bias} -> [O (BHSD), LSE (BHS f32)].
    dispatch.mojo:380-415: B,S,H,D from the BSHD Q layout; has_bias defaults to True."""
    q_layout = node.src(0).layout()
    B, S, H, D = (q_layout.shape(i) for i in range(4))
    scale = float(node.attrs()["scale"])
    is_causal = bool(node.attrs()["is_causal"])
    has_bias = bool(node.attrs().get("has_bias", True))
    _require_float(node.dtype(), "flash_attn_fwd")
    dst = AnyBuffer.create(node.dtype(), device, node.numel())
    lse = AnyBuffer.create(F32, device, B * H * S)
    # {layout: "bshd"} (set by fuse_attention_output_layout): O is written (B, S, H, D) like Q
    fwd = device.lib.mg_flash_attn_fwd_bshd if node.attrs().get("layout") == "bshd" else device.lib.mg_flash_attn_fwd
    fwd(inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), inputs[3].data_ptr(), dst.data_ptr(),
        lse.data_ptr(), B, S, H, D, scale, int(is_causal), int(has_bias), node.dtype(), device.stream)
    return [dst, lse]


def flash_attn_bwd_sched(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """FLASH_ATTN_GRAD[dO, O, Q, K, V, mask, LSE] -> [dQ, dK, dV].
    dispatch.mojo:441-481: has_bias defaults to `not is_causal`."""
    q_layout = node.src(2).layout()
    B, S, H, D = (q_layout.shape(i) for i in range(4))
    scale = float(node.attrs()["scale"])
    is_causal = bool(node.attrs()["is_causal"])
    has_bias = bool(node.attrs().get("has_bias", not is_causal))
    numel = q_layout.numel()
    _require_float(node.dtype(), "flash_attn_bwd")
    dq = AnyBuffer.create(node.dtype(), device, numel)
    dk = AnyBuffer.create(node.dtype(), device, numel)
    dv = AnyBuffer.create(node.dtype(), device, numel)
    bwd = device.lib.mg_flash_attn_bwd_bshd if node.attrs().get("layout") == "bshd" else device.lib.mg_flash_attn_bwd
    bwd(*(inputs[i].data_ptr() for i in range(7)), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, S, H, D, scale,
        int(is_causal), int(has_bias), node.dtype(), device.stream)
    return [dq, dk, dv]


def _i64_array(values: Sequence[int]):
    return (C.c_int64 * len(values))(*values)


def cross_entropy(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """CROSS_ENTROPY[logits, labels] -> (1,).  runtime/__init__.mojo:530-533:
    contiguous operands take the flat kernel, anything else the strided one."""
    la = node.src(0).layout()
    lb = node.src(1).layout()
    _require_float(node.dtype(), "cross_entropy")
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    C_ = la.shape(la.rank() - 1)
    N = la.numel() // C_
    if la.is_contiguous() and lb.is_contiguous():
        device.lib.mg_cross_entropy(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), N, C_, node.dtype(),
                                    device.stream)
    else:
        device.lib.mg_cross_entropy_strided(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), la.rank(),
                                            _i64_array(la.shape()), _i64_array(la.stride()),
                                            _i64_array(lb.stride()), node.dtype(), device.stream)
    return [out]


def cross_entropy_grad(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """CROSS_ENTROPY_GRAD[logits, labels, upstream].  runtime/__init__.mojo:563-580."""
    la = node.src(0).layout()
    lb = node.src(1).layout()
    _require_float(node.dtype(), "cross_entropy_grad")
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    C_ = la.shape(la.rank() - 1)
    N = la.numel() // C_
    if la.is_contiguous() and lb.is_contiguous():
        device.lib.mg_cross_entropy_grad(inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                                         out.data_ptr(), N, C_, node.dtype(), device.stream)
    else:
        device.lib.mg_cross_entropy_grad_strided(inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                                                 out.data_ptr(), la.rank(), _i64_array(la.shape()),
                                                 _i64_array(la.stride()), _i64_array(lb.stride()), node.dtype(),
                                                 device.stream)
    return [out]


def _matmul_dims(la: Layout, lb: Layout, N: int, b_is_nk: bool, who: str):
    """kernels/__init__.mojo:629-644,700-715,774-786."""
    rank = la.rank()
    if not (la.batch_dims_collapsible() and lb.batch_dims_collapsible()):
        raise MogradError(1, f"{who}: received non-collapsible batch dims, expected op.mojo to materialise these first")
    M = la.shape(rank - 2)
    K = la.shape(rank - 1)
    lda0, lda1 = la.stride(rank - 2), la.stride(rank - 1)
    ldb0, ldb1 = lb.stride(lb.rank() - 2), lb.stride(lb.rank() - 1)
    batch = la.numel() // (M * K)
    bsa = la.stride(rank - 3) if rank >= 3 else M * K
    bsb = lb.stride(lb.rank() - 3) if lb.rank() >= 3 else (N * K if b_is_nk else K * N)
    return batch, M, K, lda0, lda1, ldb0, ldb1, bsa, bsb


def matmul(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """MATMUL[A (.., M, K), B (.., K, N)].  dispatch.mojo:227-244."""
    la, lb = node.src(0).layout(), node.src(1).layout()
    N = node.shape(node.layout().rank() - 1)
    batch, M, K, lda0, lda1, ldb0, ldb1, bsa, bsb = _matmul_dims(la, lb, N, False, "matmul")
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_matmul(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), batch, M, N, K, lda0, lda1,
                         ldb0, ldb1, bsa, bsb, node.dtype(), device.stream)
    return [out]


def matmul_t(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """MATMUL_BT[A (.., M, K), B (.., N, K)] = A B^T.  dispatch.mojo:227-244."""
    la, lb = node.src(0).layout(), node.src(1).layout()
    N = node.shape(node.layout().rank() - 1)
    batch, M, K, lda0, lda1, ldb0, ldb1, bsa, bsb = _matmul_dims(la, lb, N, True, "matmul")
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_matmul_bt(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), batch, M, N, K, lda0, lda1,
                            ldb0, ldb1, bsa, bsb, node.dtype(), device.stream)
    return [out]


def matmul_bias_bt(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """MATMUL_BIAS_BT[A, B (N, K), bias (N)] = A B^T + bias.  dispatch.mojo:260-278."""
    la, lb = node.src(0).layout(), node.src(1).layout()
    N = node.shape(node.layout().rank() - 1)
    batch, M, K, lda0, lda1, ldb0, ldb1, bsa, bsb = _matmul_dims(la, lb, N, True, "matmul_bias")
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_matmul_bias_bt(inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), out.data_ptr(),
                                 batch, M, N, K, lda0, lda1, ldb0, ldb1, bsa, bsb, node.dtype(), device.stream)
    return [out]


def sum(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:  # noqa: A001 (reference name)
    """SUM{axis}.  runtime/__init__.mojo:390-393, dispatch.mojo:196-212.  Only the axis
    form over a contiguous source is on this path (db = dY.sum(0))."""
    if "axis" not in node.attrs():
        raise MogradError(2, "sum: the full reduction is outside the backward hot path")
    layout = node.src(0).layout()
    inputs = _materialise(node, inputs, device, 1)
    outer, reduce_size, inner = layout.reduce_dims(int(node.attrs()["axis"]))
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_sum_axis(inputs[0].data_ptr(), out.data_ptr(), outer, reduce_size, inner, node.dtype(),
                           device.stream)
    return [out]


def relu_grad(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """RELU_GRAD[relu_out, upstream].  runtime/__init__.mojo:351-352."""
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    if _flat(node, inputs, 2):
        device.lib.mg_relu_grad(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), node.numel(), node.dtype(),
                                device.stream)
    else:
        la, lb = node.src(0).layout(), node.src(1).layout()
        device.lib.mg_relu_grad_strided(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), la.rank(),
                                        _i64_array(la.shape()), _i64_array(la.stride()), _i64_array(lb.stride()),
                                        node.dtype(), device.stream)
    return [out]


def _materialise(node: Node, inputs: List[AnyBuffer], device: Device, count: int) -> List[AnyBuffer]:
    """The first `count` operands as contiguous buffers.  The reference reads strided views
    element by element inside each kernel (`*_strided` exports, kernels/strided.mojo).  Here add,
    relu, relu_grad, cast and softmax have strided entries of their own; the kernels that use this
    helper (softmax_grad, argmax, axis sums, scatter_add) copy a strided operand row-major with
    mg_contiguous first and run the contiguous kernel on the copy: same values, one extra
    pass for the rare strided case."""
    out = list(inputs)
    for i in range(count):
        layout = node.src(i).layout()
        if layout.is_contiguous():
            continue
        dtype = node.src(i).dtype()
        tmp = AnyBuffer.create(dtype, device, layout.numel())
        device.lib.mg_contiguous(inputs[i].data_ptr(), tmp.data_ptr(), layout.rank(), _i64_array(layout.shape()),
                                 _i64_array(layout.stride()), dtype, device.stream)
        out[i] = tmp
    return out


def _flat(node: Node, inputs: List[AnyBuffer], count: int) -> bool:
    """Whether the first `count` operands can take a flat kernel: contiguous, and starting on the
    16-byte boundary those kernels read from (a view into the middle of a buffer may not)."""
    return all(node.src(i).layout().is_contiguous() and (inputs[i].data_ptr().value or 0) % 16 == 0
               for i in range(count))


def add(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """ADD[a, b] (residual connections, gradient accumulation, a broadcast bias).
    runtime/__init__.mojo:319-333: contiguous operands take the flat kernel, views the strided one."""
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    if _flat(node, inputs, 2):
        device.lib.mg_add(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), node.numel(), node.dtype(),
                          device.stream)
    else:
        la, lb = node.src(0).layout(), node.src(1).layout()
        device.lib.mg_add_strided(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), la.rank(),
                                  _i64_array(la.shape()), _i64_array(la.stride()), _i64_array(lb.stride()),
                                  node.dtype(), device.stream)
    return [out]


def relu(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """RELU[a].  runtime/__init__.mojo:296-297."""
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    layout = node.src(0).layout()
    if _flat(node, inputs, 1):
        device.lib.mg_relu(inputs[0].data_ptr(), out.data_ptr(), node.numel(), node.dtype(), device.stream)
    else:
        device.lib.mg_relu_strided(inputs[0].data_ptr(), out.data_ptr(), layout.rank(), _i64_array(layout.shape()),
                                   _i64_array(layout.stride()), node.dtype(), device.stream)
    return [out]


def cast(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """CAST[a] to node.dtype().  runtime/__init__.mojo:300-311."""
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    layout = node.src(0).layout()
    if _flat(node, inputs, 1):
        device.lib.mg_cast(inputs[0].data_ptr(), out.data_ptr(), node.numel(), node.src(0).dtype(), node.dtype(),
                           device.stream)
    else:
        device.lib.mg_cast_strided(inputs[0].data_ptr(), out.data_ptr(), layout.rank(), _i64_array(layout.shape()),
                                   _i64_array(layout.stride()), node.src(0).dtype(), node.dtype(), device.stream)
    return [out]


def contiguous(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """CONTIGUOUS[a]: row-major copy of a strided view.  runtime/__init__.mojo:456-461."""
    layout = node.src(0).layout()
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_contiguous(inputs[0].data_ptr(), out.data_ptr(), layout.rank(), _i64_array(layout.shape()),
                             _i64_array(layout.stride()), node.dtype(), device.stream)
    return [out]


def gather(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """GATHER[src (rows, row_size), indices] -> (*indices.shape, row_size).
    runtime/__init__.mojo:239-240, kernels/__init__.mojo:132-163."""
    la = node.src(0).layout()
    lb = node.src(1).layout()
    if la.rank() != 2:  # op.mojo:367-368
        raise MogradError(1, "gather expects a 2D source tensor [num_rows, row_size]")
    if not lb.is_contiguous():  # strided indices: copy them row-major first
        idx = AnyBuffer.create(node.src(1).dtype(), device, lb.numel())
        device.lib.mg_contiguous(inputs[1].data_ptr(), idx.data_ptr(), lb.rank(), _i64_array(lb.shape()),
                                 _i64_array(lb.stride()), node.src(1).dtype(), device.stream)
        inputs = [inputs[0], idx]
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_gather(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), lb.numel(), la.shape(0),
                         la.shape(1), la.stride(0), la.stride(1), node.src(1).dtype(), node.dtype(), device.stream)
    return [out]


def scatter_add(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """SCATTER_ADD[indices, values (*indices.shape, row_size)] -> (num_rows, row_size).
    runtime/__init__.mojo:243-256; the output needs no zero fill here."""
    la = node.src(0).layout()
    lb = node.src(1).layout()
    if lb.rank() != la.rank() + 1:  # op.mojo:375-376
        raise MogradError(1, "scatter_add expects values shaped [*indices.shape, row_size]")
    inputs = _materialise(node, inputs, device, 2)
    row_size = lb.shape(lb.rank() - 1)
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    if device.pending is not None:
        device.lib.mg_scatter_add_deferred(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), la.numel(),
                                           node.shape(0), row_size, node.src(0).dtype(), node.dtype(), node.dtype(),
                                           device.pending, device.stream)
    else:
        device.lib.mg_scatter_add(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), la.numel(),
                                  node.shape(0), row_size, node.src(0).dtype(), node.dtype(), device.stream)
    return [out]


def softmax(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """SOFTMAX[a] over the last axis.  runtime/__init__.mojo (softmax), kernels/__init__.mojo:1015-1030."""
    layout = node.src(0).layout()
    _require_float(node.dtype(), "softmax")
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    if layout.is_contiguous():
        cols = layout.shape(layout.rank() - 1)
        rows = layout.numel() // cols if cols else 0
        device.lib.mg_softmax(inputs[0].data_ptr(), out.data_ptr(), rows, cols, node.dtype(), device.stream)
    else:  # kernels/__init__.mojo:1033-1060: views go to the strided kernel
        device.lib.mg_softmax_strided(inputs[0].data_ptr(), out.data_ptr(), layout.rank(), _i64_array(layout.shape()),
                                      _i64_array(layout.stride()), node.dtype(), device.stream)
    return [out]


def softmax_grad(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """SOFTMAX_GRAD[y, upstream] (mograd/grad.mojo:232-234).  kernels/__init__.mojo:1062-1090."""
    la = node.src(0).layout()
    inputs = _materialise(node, inputs, device, 2)
    _require_float(node.dtype(), "softmax_grad")
    size = la.shape(la.rank() - 1)
    N = la.numel() // size
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_softmax_grad(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), N, size, node.dtype(),
                               device.stream)
    return [out]


def argmax(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """ARGMAX{axis}: index of the first largest value, stored in the tensor's float dtype.
    runtime/__init__.mojo:402-405; without `axis` the whole tensor is one lane."""
    layout = node.src(0).layout()
    inputs = _materialise(node, inputs, device, 1)
    _require_float(node.dtype(), "argmax")
    if "axis" in node.attrs():
        outer, reduce_size, inner = layout.reduce_dims(int(node.attrs()["axis"]))
    else:
        outer, reduce_size, inner = 1, layout.numel(), 1
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_argmax_axis(inputs[0].data_ptr(), out.data_ptr(), outer, reduce_size, inner, node.dtype(),
                              device.stream)
    return [out]


# --------------------------------------------------------------------------- #
# Exec functions for the fused nodes that the gradient rules below emit.  The reference has
# no counterpart for them: its Linear backward is matmul_grad + transpose_grad + expand_grad
# (mograd/grad.mojo:180-187,278-288), its LAYER_NORM has one output
# (mograd/runtime/__init__.mojo:425-426) and its labels are dense.  They follow the pattern
# of its multi-output FLASH_ATTN / FLASH_ATTN_GRAD pair (mograd/grad.mojo:309-344).
# --------------------------------------------------------------------------- #


def linear_bwd(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """LINEAR_GRAD[dY (.., N), X (.., K), W (N, K)(, prior)]{has_bias, relu_mask, accumulate}
    -> [dX (.., K), dW (N, K), db (N)] for Y = X W^T (+ b): dX = dY W, dW = dY^T X written in W's
    layout, db = column sums of dY (two results without has_bias).  relu_mask: X is a ReLU's
    output and dX is zeroed where X <= 0 (the RELU_GRAD of the layer below, folded in);
    accumulate: dX = prior + dY W with `prior` the fourth source.  Leading dimensions collapse
    into the row count."""
    ldy, lx, lw = (node.src(i).layout() for i in range(3))
    accumulate = bool(node.attrs().get("accumulate", False))
    relu_mask = bool(node.attrs().get("relu_mask", False))
    inputs = _materialise(node, inputs, device, 4 if accumulate else 3)
    _require_float(node.dtype(), "linear_bwd")
    N, K = lw.shape(0), lw.shape(1)
    M = lx.numel() // K
    if ldy.numel() != M * N or lw.rank() != 2:
        raise MogradError(1, "linear_bwd: dY, X and W do not describe Y = X W^T")
    has_bias = bool(node.attrs().get("has_bias", True))
    dx = AnyBuffer.create(node.dtype(), device, M * K)
    if accumulate:  # the kernel adds into dx: start it from the prior gradient
        device.lib.mg_copy_device(dx.data_ptr(), inputs[3].data_ptr(), dx.size_bytes(), device.stream)
    dw = AnyBuffer.create(node.dtype(), device, N * K)
    db = AnyBuffer.create(node.dtype(), device, N) if has_bias else None
    args = (inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), dx.data_ptr(), dw.data_ptr(),
            db.data_ptr() if has_bias else None, M, N, K)
    if device.pending is not None:
        device.lib.mg_linear_bwd_deferred(*args, int(accumulate), int(relu_mask), node.dtype(), node.dtype(),
                                          device.pending, device.stream)
    elif accumulate or relu_mask:
        device.lib.mg_linear_bwd_fused(*args, int(accumulate), int(relu_mask), node.dtype(), device.stream)
    else:
        device.lib.mg_linear_bwd(*args, node.dtype(), device.stream)
    return [dx, dw, db] if has_bias else [dx, dw]


def layer_norm_fwd_stats(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """LAYER_NORM_STATS[x, gamma, beta]{eps} -> [y, mean (rows) f32, rstd (rows) f32]: the
    forward as a multi-output node, so that the backward reuses the row statistics."""
    x_layout = node.src(0).layout()
    cols = x_layout.shape(x_layout.rank() - 1)
    rows = x_layout.numel() // cols
    _require_float(node.dtype(), "layer_norm_fwd_stats")
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    mean = AnyBuffer.create(F32, device, rows)
    rstd = AnyBuffer.create(F32, device, rows)
    device.lib.mg_layer_norm_fwd_stats(inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                                       out.data_ptr(), mean.data_ptr(), rstd.data_ptr(), rows, cols,
                                       float(node.attrs()["eps"]), node.dtype(), device.stream)
    return [out, mean, rstd]


def layer_norm_bwd_stats(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """LAYER_NORM_STATS_GRAD[dy, x, gamma, mean, rstd] -> [dx, dgamma, dbeta], and
    LAYER_NORM_STATS_GRAD_ADD[dy, x, gamma, mean, rstd, residual]: dx = gradient + residual (the
    gradient that reaches x along another path, e.g. a skip connection)."""
    x_layout = node.src(1).layout()
    gamma_layout = node.src(2).layout()
    cols = x_layout.shape(x_layout.rank() - 1)
    rows = x_layout.numel() // cols
    _require_float(node.dtype(), "layer_norm_bwd_stats")
    with_residual = node.op_type == "LAYER_NORM_STATS_GRAD_ADD"
    if with_residual:
        inputs = _materialise(node, inputs, device, 6)
    dx = AnyBuffer.create(node.dtype(), device, x_layout.numel())
    dgamma = AnyBuffer.create(node.dtype(), device, gamma_layout.numel())
    dbeta = AnyBuffer.create(node.dtype(), device, gamma_layout.numel())
    residual = inputs[5].data_ptr() if with_residual else None
    ptrs = [inputs[i].data_ptr() for i in range(5)]
    if device.pending is not None:
        device.lib.mg_layer_norm_bwd_stats_deferred(*ptrs, residual, dx.data_ptr(), dgamma.data_ptr(), dbeta.data_ptr(),
                                                    rows, cols, node.dtype(), node.dtype(), device.pending, device.stream)
    elif with_residual:
        device.lib.mg_layer_norm_bwd_stats_add(*ptrs, residual, dx.data_ptr(), dgamma.data_ptr(), dbeta.data_ptr(), rows,
                                               cols, node.dtype(), device.stream)
    else:
        device.lib.mg_layer_norm_bwd_stats(*ptrs, dx.data_ptr(), dgamma.data_ptr(), dbeta.data_ptr(), rows, cols,
                                           node.dtype(), device.stream)
    return [dx, dgamma, dbeta]


def linear_layer_norm_bwd(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """LINEAR_LAYER_NORM_GRAD[dY (.., N), x (.., K), W (N, K), h (.., K), gamma, mean, rstd(, prior)]{has_bias,
    accumulate} -> [dh, dgamma, dbeta, dW, db] for Y = x W^T (+ b) with x = LayerNorm(h): the
    LINEAR_GRAD of the layer and the LAYER_NORM_STATS_GRAD(_ADD) of the LayerNorm that feeds it as
    one node (mg_linear_bwd_layer_norm_bwd), dY W never stored.  accumulate: dh = prior + the
    LayerNorm's input gradient, `prior` the eighth source."""
    ldy, lx, lw = (node.src(i).layout() for i in range(3))
    accumulate = bool(node.attrs().get("accumulate", False))
    has_bias = bool(node.attrs().get("has_bias", True))
    inputs = _materialise(node, inputs, device, 8 if accumulate else 7)
    _require_float(node.dtype(), "linear_layer_norm_bwd")
    N, K = lw.shape(0), lw.shape(1)
    M = lx.numel() // K
    if ldy.numel() != M * N or lw.rank() != 2 or node.src(3).layout().numel() != M * K:
        raise MogradError(1, "linear_layer_norm_bwd: dY, x, W and h do not describe Y = LayerNorm(h) W^T")
    dh = AnyBuffer.create(node.dtype(), device, M * K)
    if accumulate:  # the kernel adds into dh: start it from the prior gradient
        device.lib.mg_copy_device(dh.data_ptr(), inputs[7].data_ptr(), dh.size_bytes(), device.stream)
    dgamma = AnyBuffer.create(node.dtype(), device, K)
    dbeta = AnyBuffer.create(node.dtype(), device, K)
    dw = AnyBuffer.create(node.dtype(), device, N * K)
    db = AnyBuffer.create(node.dtype(), device, N) if has_bias else None
    device.lib.mg_linear_bwd_layer_norm_bwd(*(inputs[i].data_ptr() for i in range(7)), dh.data_ptr(), dw.data_ptr(),
                                            db.data_ptr() if has_bias else None, dgamma.data_ptr(), dbeta.data_ptr(),
                                            M, N, K, int(accumulate), node.dtype(), node.dtype(), device.pending,
                                            device.stream)
    return [dh, dgamma, dbeta, dw, db] if has_bias else [dh, dgamma, dbeta, dw]


def matmul_bt_add(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """MATMUL_BT_ADD[A, B (N, K), R] = A B^T + R (R laid out like the result): the residual
    addition of a transformer block on the product that feeds it."""
    la, lb = node.src(0).layout(), node.src(1).layout()
    N = node.shape(node.layout().rank() - 1)
    batch, M, K, lda0, lda1, ldb0, ldb1, bsa, bsb = _matmul_dims(la, lb, N, True, "matmul")
    residual = inputs[2]
    if not node.src(2).layout().is_contiguous():
        residual = _materialise(Node("ADD", node.layout(), node.dtype(), [node.src(2)]), [inputs[2]], device, 1)[0]
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_matmul_bt_add(inputs[0].data_ptr(), inputs[1].data_ptr(), residual.data_ptr(), out.data_ptr(), batch, M,
                                N, K, lda0, lda1, ldb0, ldb1, bsa, bsb, node.dtype(), device.stream)
    return [out]


def matmul_bias_relu_bt(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """MATMUL_BIAS_RELU_BT[A, B (N, K), bias (N)] = max(A B^T + bias, 0)."""
    la, lb = node.src(0).layout(), node.src(1).layout()
    N = node.shape(node.layout().rank() - 1)
    batch, M, K, lda0, lda1, ldb0, ldb1, bsa, bsb = _matmul_dims(la, lb, N, True, "matmul_bias")
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_matmul_bias_relu_bt(inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), out.data_ptr(),
                                      batch, M, N, K, lda0, lda1, ldb0, ldb1, bsa, bsb, node.dtype(), device.stream)
    return [out]


def reshape(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """RESHAPE[a]: a contiguous tensor under another shape, a view (mograd/op.mojo:335-337 folds
    the identity; a strided source is materialised first, like the reference's reshape)."""
    (src,) = _materialise(node, inputs, device, 1)
    return [src.view(Layout(*node.layout().shape(), base_offset=src.offset_elems))]


def transpose(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """TRANSPOSE[a]{dim0, dim1}: a strided view of the same storage (runtime/__init__.mojo:157)."""
    return [inputs[0].view(node.layout())]


def expand(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """EXPAND[a]: a broadcast view, stride 0 along the expanded axes (runtime/__init__.mojo, the view
    ops; grad.mojo:156-177 builds it as the gradient of SUM).  A consumer that needs rows in memory
    materialises it with mg_contiguous, which reads stride-0 views."""
    return [inputs[0].view(node.layout())]


def flash_attn_packed_fwd(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """FLASH_ATTN_PACKED[qkv (B, S, 3, H, D), mask]{scale, is_causal, has_bias} -> [O (B, S, H, D),
    LSE (B, H, S) f32]: Q, K and V are the three slices of one projection's output, and O comes out
    in the layout the next projection reads."""
    B, S, three, H, D = (node.src(0).layout().shape(i) for i in range(5))
    if three != 3:
        raise MogradError(1, "flash_attn_packed: qkv must be (B, S, 3, H, D)")
    is_causal = bool(node.attrs()["is_causal"])
    has_bias = bool(node.attrs().get("has_bias", True))
    _require_float(node.dtype(), "flash_attn_fwd")
    dst = AnyBuffer.create(node.dtype(), device, node.numel())
    lse = AnyBuffer.create(F32, device, B * H * S)
    mask = inputs[1].data_ptr() if len(inputs) > 1 else None
    device.lib.mg_flash_attn_fwd_packed(inputs[0].data_ptr(), mask, dst.data_ptr(), lse.data_ptr(), B, S, H, D,
                                        float(node.attrs()["scale"]), int(is_causal), int(has_bias), node.dtype(),
                                        device.stream)
    return [dst, lse]


def flash_attn_packed_bwd(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """FLASH_ATTN_PACKED_GRAD[dO, O, qkv, LSE(, mask)] -> dqkv (B, S, 3, H, D)."""
    B, S, _, H, D = (node.src(2).layout().shape(i) for i in range(5))
    is_causal = bool(node.attrs()["is_causal"])
    has_bias = bool(node.attrs().get("has_bias", not is_causal))
    _require_float(node.dtype(), "flash_attn_bwd")
    inputs = _materialise(node, inputs, device, 1)  # dO contiguous, as flash_attn_grad makes it
    dqkv = AnyBuffer.create(node.dtype(), device, node.numel())
    mask = inputs[4].data_ptr() if len(inputs) > 4 else None
    device.lib.mg_flash_attn_bwd_packed(inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(), mask,
                                        inputs[3].data_ptr(), dqkv.data_ptr(), B, S, H, D, float(node.attrs()["scale"]),
                                        int(is_causal), int(has_bias), node.dtype(), device.stream)
    return [dqkv]


def cross_entropy_ids(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """CROSS_ENTROPY_IDS[logits (.., C), ids (..) int32/int64] -> (1,): labels as class ids
    instead of the reference's one_hot(...).cast(f32) rows."""
    la = node.src(0).layout()
    inputs = _materialise(node, inputs, device, 2)
    _require_float(node.dtype(), "cross_entropy_ids")
    C_ = la.shape(la.rank() - 1)
    N = la.numel() // C_
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_cross_entropy_ids(inputs[0].data_ptr(), inputs[1].data_ptr(), out.data_ptr(), N, C_, node.dtype(),
                                    node.src(1).dtype(), device.stream)
    return [out]


def cross_entropy_grad_ids(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """CROSS_ENTROPY_IDS_GRAD[logits, ids, upstream (1,)] -> dlogits."""
    la = node.src(0).layout()
    inputs = _materialise(node, inputs, device, 2)
    _require_float(node.dtype(), "cross_entropy_grad_ids")
    C_ = la.shape(la.rank() - 1)
    N = la.numel() // C_
    out = AnyBuffer.create(node.dtype(), device, node.numel())
    device.lib.mg_cross_entropy_grad_ids(inputs[0].data_ptr(), inputs[1].data_ptr(), inputs[2].data_ptr(),
                                         out.data_ptr(), N, C_, node.dtype(), node.src(1).dtype(), device.stream)
    return [out]


# Op type -> exec function, the rows of the reference's rule table that belong to this
# path (mograd/runtime/__init__.mojo:113-167).
SCHEDULER_RULES = {
    "ADD": add,
    "RELU": relu,
    "CAST": cast,
    "CONTIGUOUS": contiguous,
    "GATHER": gather,
    "SCATTER_ADD": scatter_add,
    "RELU_GRAD": relu_grad,
    "SOFTMAX": softmax,
    "SOFTMAX_GRAD": softmax_grad,
    "ARGMAX": argmax,
    "SUM": sum,
    "MATMUL": matmul,
    "MATMUL_BT": matmul_t,
    "MATMUL_BIAS_BT": matmul_bias_bt,
    "LAYER_NORM": layer_norm_fwd,
    "LAYER_NORM_GRAD": layer_norm_bwd,
    "FLASH_ATTN": flash_attn_fwd_sched,
    "FLASH_ATTN_GRAD": flash_attn_bwd_sched,
    "CROSS_ENTROPY": cross_entropy,
    "CROSS_ENTROPY_GRAD": cross_entropy_grad,
    # fused nodes emitted by GRAD_RULES below (no counterpart in the reference's table)
    "LINEAR_GRAD": linear_bwd,
    "LAYER_NORM_STATS": layer_norm_fwd_stats,
    "LAYER_NORM_STATS_GRAD": layer_norm_bwd_stats,
    "CROSS_ENTROPY_IDS": cross_entropy_ids,
    "CROSS_ENTROPY_IDS_GRAD": cross_entropy_grad_ids,
    # views, and the fused nodes that mograd_amd.rewrites.GPU_REWRITES creates
    "RESHAPE": reshape,
    "TRANSPOSE": transpose,
    "EXPAND": expand,
    "MATMUL_BT_ADD": matmul_bt_add,
    "MATMUL_BIAS_RELU_BT": matmul_bias_relu_bt,
    "LAYER_NORM_STATS_GRAD_ADD": layer_norm_bwd_stats,
    "LINEAR_LAYER_NORM_GRAD": linear_layer_norm_bwd,
    "FLASH_ATTN_PACKED": flash_attn_packed_fwd,
    "FLASH_ATTN_PACKED_GRAD": flash_attn_packed_bwd,
}


def run(node: Node, inputs: List[AnyBuffer], device: Device) -> List[AnyBuffer]:
    """One scheduler step: first matching rule wins (pattern_matcher.mojo:74-80)."""
    try:
        fn = SCHEDULER_RULES[node.op_type]
    except KeyError:
        raise MogradError(2, f"no scheduler rule for op {node.op_type} on the backward hot path") from None
    return fn(node, inputs, device)


# --------------------------------------------------------------------------- #
# Gradient rules: node + upstream -> one gradient node per source (None: no gradient edge),
# the GradFn of mograd/grad.mojo:12.  The rules of the reference that lie on this path are
# restated (layer_norm_grad :296-306, flash_attn_grad :309-344, cross_entropy_grad :224-230,
# gettuple_grad :291-293); the others are the rules it lacks (mograd/grad.mojo:30-65 has
# none for MATMUL_BT / MATMUL_BIAS_BT, so its Linear backward is three separate products and
# a reduction over an unsimplified graph): each emits one multi-output node whose results
# GETTUPLE selects, the way the reference treats LAYER_NORM_GRAD and FLASH_ATTN_GRAD.
# --------------------------------------------------------------------------- #


def _gettuple(src: Node, index: int, layout: Layout, dtype: int) -> Node:
    return Node("GETTUPLE", layout, dtype, [src], {"index": index})


def _rows_layout(layout: Layout) -> Layout:
    cols = layout.shape(layout.rank() - 1)
    return Layout(layout.numel() // cols)


def linear_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """MATMUL_BIAS_BT[X, W, b] or MATMUL_BT[X, W] -> LINEAR_GRAD[dY, X, W] -> dX, dW(, db)."""
    x, w = node.src(0), node.src(1)
    has_bias = node.op_type == "MATMUL_BIAS_BT"
    bwd = Node("LINEAR_GRAD", x.layout().as_contiguous(), x.dtype(), [upstream, x, w], {"has_bias": has_bias})
    grads: List[Optional[Node]] = [_gettuple(bwd, 0, x.layout().as_contiguous(), x.dtype()),
                                   _gettuple(bwd, 1, w.layout().as_contiguous(), w.dtype())]
    if has_bias:
        b = node.src(2)
        grads.append(_gettuple(bwd, 2, b.layout().as_contiguous(), b.dtype()))
    return grads


def layer_norm_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:296-306."""
    x, gamma = node.src(0), node.src(1)
    bwd = Node("LAYER_NORM_GRAD", x.layout().as_contiguous(), x.dtype(), [upstream, x, gamma], dict(node.attrs()))
    return [_gettuple(bwd, 0, x.layout().as_contiguous(), x.dtype()),
            _gettuple(bwd, 1, gamma.layout().as_contiguous(), gamma.dtype()),
            _gettuple(bwd, 2, gamma.layout().as_contiguous(), gamma.dtype())]


def layer_norm_stats_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """LAYER_NORM_STATS[x, gamma, beta] (outputs y, mean, rstd; `upstream` is dy, passed through
    GETTUPLE 0 by gettuple_grad) -> LAYER_NORM_STATS_GRAD[dy, x, gamma, mean, rstd]."""
    x, gamma = node.src(0), node.src(1)
    rows = _rows_layout(x.layout())
    mean = _gettuple(node, 1, rows, F32)
    rstd = _gettuple(node, 2, rows, F32)
    bwd = Node("LAYER_NORM_STATS_GRAD", x.layout().as_contiguous(), x.dtype(), [upstream, x, gamma, mean, rstd])
    return [_gettuple(bwd, 0, x.layout().as_contiguous(), x.dtype()),
            _gettuple(bwd, 1, gamma.layout().as_contiguous(), gamma.dtype()),
            _gettuple(bwd, 2, gamma.layout().as_contiguous(), gamma.dtype())]


def flash_attn_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:309-344: O and LSE from the forward's two outputs, LSE (B,H,S) f32."""
    q, k, v, mask = (node.src(i) for i in range(4))
    B, S, H = q.layout().shape(0), q.layout().shape(1), q.layout().shape(2)
    o = _gettuple(node, 0, node.layout(), node.dtype())
    lse = _gettuple(node, 1, Layout(B, H, S), F32)
    d_o = upstream if upstream.layout().is_contiguous() else Node("CONTIGUOUS", upstream.layout().as_contiguous(),
                                                                  upstream.dtype(), [upstream])
    bwd = Node("FLASH_ATTN_GRAD", q.layout().as_contiguous(), q.dtype(), [d_o, o, q, k, v, mask, lse], dict(node.attrs()))
    return [_gettuple(bwd, i, t.layout().as_contiguous(), t.dtype()) for i, t in enumerate((q, k, v))] + [None]


def cross_entropy_grad_rule(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:224-230, and its class-id form."""
    logits, labels = node.src(0), node.src(1)
    op = "CROSS_ENTROPY_IDS_GRAD" if node.op_type == "CROSS_ENTROPY_IDS" else "CROSS_ENTROPY_GRAD"
    return [Node(op, logits.layout().as_contiguous(), logits.dtype(), [logits, labels, upstream]), None]


def relu_grad_rule(node: Node, upstream: Node) -> List[Optional[Node]]:
    """relu_grad: RELU_GRAD[relu_out, upstream]."""
    return [Node("RELU_GRAD", node.layout().as_contiguous(), node.dtype(), [node, upstream])]


def gettuple_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:291-293: the upstream passes through to the multi-output source."""
    return [upstream]


def add_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:126-127: both sources receive the upstream (same shapes on this path;
    the reference's un-broadcast of an EXPAND source is expand_grad, outside it)."""
    for src in node.srcs:
        if src.layout().shape() != node.layout().shape():
            raise MogradError(2, "add_grad: broadcast operands are outside the backward hot path")
    return [upstream, upstream]


def contiguous_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:269: a copy's gradient is the upstream itself."""
    return [upstream]


def cast_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:237: the upstream cast back to the source's dtype."""
    src = node.src(0)
    if src.dtype() not in (F32, F16, BF16):
        return [None]
    return [Node("CAST", upstream.layout().as_contiguous(), src.dtype(), [upstream])]


def gather_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:190: SCATTER_ADD[indices, upstream] in the table's shape; no gradient for
    the indices."""
    table, indices = node.src(0), node.src(1)
    return [Node("SCATTER_ADD", table.layout().as_contiguous(), table.dtype(), [indices, upstream]), None]


def softmax_grad_rule(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:232-234: SOFTMAX_GRAD[y, upstream]."""
    return [Node("SOFTMAX_GRAD", node.layout().as_contiguous(), node.dtype(), [node, upstream])]


def sum_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:156-177: the upstream broadcast back over the summed axis, an EXPAND view
    with stride 0 there (every stride 0 for the full reduction)."""
    shape = node.src(0).layout().shape()
    up = upstream.layout()
    if "axis" not in node.attrs():
        strides = [0] * len(shape)
    else:
        ax = int(node.attrs()["axis"]) % len(shape)
        if up.rank() == len(shape):  # keepdim: the size-1 axis is expanded in place
            strides = [0 if i == ax else up.stride(i) for i in range(len(shape))]
        else:
            strides = list(up.stride())
            strides.insert(ax, 0)
    return [Node("EXPAND", Layout(*shape, strides=strides, base_offset=up.base_offset), node.dtype(), [upstream])]


def expand_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:278-288: the upstream summed over the leading axes that EXPAND added and,
    keeping the dimension, over every axis it widened."""
    src, out = node.src(0).layout(), node.layout()
    grad = upstream
    for _ in range(out.rank() - src.rank()):
        dims = grad.layout().shape()
        grad = Node("SUM", Layout(*dims[1:]), grad.dtype(), [grad], {"axis": 0})
    for i in range(src.rank()):
        if src.shape(i) != grad.layout().shape(i):
            dims = list(grad.layout().shape())
            dims[i] = 1
            grad = Node("SUM", Layout(*dims), grad.dtype(), [grad], {"axis": i, "keepdim": True})
    return [grad]


def reshape_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo (reshape_grad): the upstream under the source's shape."""
    src = node.src(0)
    return [Node("RESHAPE", src.layout().as_contiguous(), upstream.dtype(), [upstream])]


def transpose_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """mograd/grad.mojo:186-187: the same two dimensions swapped back (a view)."""
    d0, d1 = int(node.attrs().get("dim0", -2)), int(node.attrs().get("dim1", -1))
    return [Node("TRANSPOSE", upstream.layout().transpose(d0, d1), upstream.dtype(), [upstream], dict(node.attrs()))]


def flash_attn_packed_grad(node: Node, upstream: Node) -> List[Optional[Node]]:
    """FLASH_ATTN_PACKED[qkv(, mask)] -> FLASH_ATTN_PACKED_GRAD[dO, O, qkv, LSE(, mask)] -> dqkv: the
    packed form of flash_attn_grad (mograd/grad.mojo:309-344); the mask gets no gradient."""
    qkv = node.src(0)
    B, S, _, H, _ = qkv.layout().shape()
    o = _gettuple(node, 0, node.layout(), node.dtype())
    lse = _gettuple(node, 1, Layout(B, H, S), F32)
    d_o = upstream if upstream.layout().is_contiguous() else Node("CONTIGUOUS", upstream.layout().as_contiguous(),
                                                                  upstream.dtype(), [upstream])
    bwd = Node("FLASH_ATTN_PACKED_GRAD", qkv.layout().as_contiguous(), qkv.dtype(), [d_o, o, qkv, lse] + node.srcs[1:],
               dict(node.attrs()))
    return [bwd] + [None] * (len(node.srcs) - 1)


GRAD_RULES = {
    "MATMUL_BT": linear_grad,
    "MATMUL_BIAS_BT": linear_grad,
    "LAYER_NORM": layer_norm_grad,
    "LAYER_NORM_STATS": layer_norm_stats_grad,
    "FLASH_ATTN": flash_attn_grad,
    "CROSS_ENTROPY": cross_entropy_grad_rule,
    "CROSS_ENTROPY_IDS": cross_entropy_grad_rule,
    "RELU": relu_grad_rule,
    "GETTUPLE": gettuple_grad,
    "ADD": add_grad,
    "CONTIGUOUS": contiguous_grad,
    "CAST": cast_grad,
    "GATHER": gather_grad,
    "SOFTMAX": softmax_grad_rule,
    "RESHAPE": reshape_grad,
    "TRANSPOSE": transpose_grad,
    "SUM": sum_grad,
    "EXPAND": expand_grad,
    "FLASH_ATTN_PACKED": flash_attn_packed_grad,
}


def _toposort(root: Node) -> List[Node]:
    """Sources before consumers, each node once (GraphUtils.toposort); iterative, so that deep
    training graphs do not run into the interpreter's recursion limit."""
    order: List[Node] = []
    seen = set()
    stack = [(root, 0)]
    seen.add(root)
    while stack:
        n, i = stack.pop()
        if i < len(n.srcs):
            stack.append((n, i + 1))
            child = n.srcs[i]
            if child not in seen:
                seen.add(child)
                stack.append((child, 0))
        else:
            order.append(n)
    return order


def gradient(root: Node, initial_grad: Node, targets: Sequence[Node]) -> List[Optional[Node]]:
    """Grad.compute (mograd/grad.mojo:22-91): walks the graph from `root` in reverse
    topological order, applies the rule of each node to its accumulated upstream and adds the
    results to its sources' gradients (ADD nodes where two paths meet).  Returns the gradient
    node of every target (None if no path reaches it)."""
    grad_map: Dict[Node, Node] = {root: initial_grad}
    for node in reversed(_toposort(root)):
        upstream = grad_map.get(node)
        if upstream is None or node.dtype() not in (F32, F16, BF16):
            continue
        rule = GRAD_RULES.get(node.op_type)
        if rule is None:
            if node.srcs:
                raise MogradError(2, f"no gradient rule for op: {node.op_type}")
            continue
        for src, g in zip(node.srcs, rule(node, upstream)):
            if g is None:
                continue
            prev = grad_map.get(src)
            grad_map[src] = g if prev is None else Node("ADD", g.layout(), g.dtype(), [prev, g])
    return [grad_map.get(t) for t in targets]


def evaluate(node: Node, device: Device) -> AnyBuffer:
    """Scheduler.run for one result (mograd/scheduler.mojo:40-80): evaluates the sources
    first, runs the node's rule once and keeps its buffers on the node; GETTUPLE selects an
    output of a multi-output source."""
    for n in _toposort(node):
        _evaluate_node(n, device)
    return node.bufs[0]


def _evaluate_node(n: Node, device: Device) -> None:
    """One node whose sources have their buffers."""
    if n.bufs is not None:
        return
    if n.op_type == "BUFFER":
        raise MogradError(1, "evaluate: a leaf node without a buffer")
    if n.op_type == "GETTUPLE":
        n.bufs = [n.src(0).bufs[int(n.attrs()["index"])]]
    else:
        n.bufs = run(n, [s_.bufs[0] for s_ in n.srcs], device)


def evaluate_many(nodes: Sequence[Node], device: Device, deferred_sums: bool = False) -> List[AnyBuffer]:
    """Scheduler.run_many (mograd/scheduler.mojo:39-82): every node of `nodes` in one walk, shared
    sub-graphs evaluated once.  With `deferred_sums` the second-stage sums of the parameter
    gradients (LINEAR_GRAD, LAYER_NORM_STATS_GRAD(_ADD), SCATTER_ADD) are left on one mg_deferred
    list and finished by a single launch after the walk: same bits, fewer launches."""
    sink = Node("SINK", Layout(1), F32, list(nodes))
    order = _toposort(sink)[:-1]
    if deferred_sums:
        pending = C.c_void_p()
        device.lib.mg_deferred_create(C.byref(pending))
        device.pending = pending
    try:
        for n in order:
            _evaluate_node(n, device)
        if deferred_sums:
            device.lib.mg_finish_deferred(device.pending, device.stream)
    finally:
        if deferred_sums:
            device.lib.mg_deferred_destroy(device.pending)
            device.pending = None
    return [n.bufs[0] for n in nodes]
