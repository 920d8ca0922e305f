"""ctypes binding of libmograd_hip.so (the C ABI declared in include/mograd_hip.h).

The library is required: there is no CPU or PyTorch fallback.  `load()` raises
`LibraryMissing` when the shared object has not been built (run
`python -m mograd_amd.build`), and every wrapped call raises `MogradError` with the
library's message on a non-zero status.
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

PKG = Path(__file__).resolve().parent
LIB_NAME = "libmograd_hip.so"

# mg_dtype
F32, F16, BF16, I32, I64 = 0, 1, 2, 3, 4
DTYPE_NAMES = {F32: "float32", F16: "float16", BF16: "bfloat16", I32: "int32", I64: "int64"}
DTYPE_SIZE = {F32: 4, F16: 2, BF16: 2, I32: 4, I64: 8}


class MogradError(RuntimeError):
    """A libmograd_hip call returned a non-zero status."""

    def __init__(self, status: int, message: str):
        super().__init__(message or f"libmograd_hip status {status}")
        self.status = status


class LibraryMissing(ImportError):
    """libmograd_hip.so is not built or cannot be loaded."""


class PoolStats(C.Structure):
    _fields_ = [
        ("allocated_bytes", C.c_int64),
        ("reserved_bytes", C.c_int64),
        ("peak_allocated", C.c_int64),
        ("peak_reserved", C.c_int64),
        ("alloc_count", C.c_int64),
        ("hit_count", C.c_int64),
        ("miss_count", C.c_int64),
        ("free_count", C.c_int64),
    ]


_p = C.c_void_p
_i = C.c_int
_l = C.c_int64
_f = C.c_float
_pl = C.POINTER(C.c_int64)

# name -> (restype, argtypes, returns_status)
PROTOTYPES = {
    "mg_version": (C.c_char_p, [], False),
    "mg_last_error": (C.c_char_p, [], False),
    "mg_init": (_i, [_i], True),
    "mg_device_cu_count": (_i, [], False),
    "mg_stream_create": (_i, [C.POINTER(_p)], True),
    "mg_stream_destroy": (_i, [_p], True),
    "mg_stream_sync": (_i, [_p], True),
    "mg_event_create": (_i, [C.POINTER(_p)], True),
    "mg_event_destroy": (_i, [_p], True),
    "mg_event_record": (_i, [_p, _p], True),
    "mg_event_elapsed_ms": (_i, [_p, _p, C.POINTER(_f)], True),
    "mg_copy_to_device": (_i, [_p, _p, _l, _p], True),
    "mg_copy_to_host": (_i, [_p, _p, _l, _p], True),
    "mg_copy_device": (_i, [_p, _p, _l, _p], True),
    "mg_fill": (_i, [_p, C.c_double, _l, _i, _p], True),
    "mg_round_class": (_l, [_l], False),
    "mg_pool_enabled": (_i, [], False),
    "mg_pool_alloc": (_i, [C.POINTER(_p), _l], True),
    "mg_pool_free": (_i, [_p], True),
    "mg_pool_empty_cache": (_i, [], True),
    "mg_pool_get_stats": (_i, [C.POINTER(PoolStats)], True),
    "mg_pool_summary": (_l, [C.c_char_p, _l], False),
    "mg_layer_norm_fwd": (_i, [_p, _p, _p, _p, _l, _l, _f, _i, _p], True),
    "mg_layer_norm_fwd_stats": (_i, [_p, _p, _p, _p, _p, _p, _l, _l, _f, _i, _p], True),
    "mg_layer_norm_bwd": (_i, [_p, _p, _p, _p, _p, _p, _l, _l, _f, _i, _p], True),
    "mg_layer_norm_bwd_stats": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _l, _l, _i, _p], True),
    "mg_layer_norm_bwd_stats_add": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _l, _l, _i, _p], True),
    "mg_cross_entropy": (_i, [_p, _p, _p, _l, _l, _i, _p], True),
    "mg_cross_entropy_grad": (_i, [_p, _p, _p, _p, _l, _l, _i, _p], True),
    "mg_cross_entropy_strided": (_i, [_p, _p, _p, _i, _pl, _pl, _pl, _i, _p], True),
    "mg_cross_entropy_grad_strided": (_i, [_p, _p, _p, _p, _i, _pl, _pl, _pl, _i, _p], True),
    "mg_cross_entropy_ids": (_i, [_p, _p, _p, _l, _l, _i, _i, _p], True),
    "mg_cross_entropy_grad_ids": (_i, [_p, _p, _p, _p, _l, _l, _i, _i, _p], True),
    "mg_cross_entropy_fused_ids": (_i, [_p, _p, _p, _p, _p, _l, _l, _i, _i, _p], True),
    "mg_cross_entropy_fused_ids_noalloc": (_i, [_p, _p, _p, _p, _p, _l, _l, _i, _i, _p], True),
    "mg_cross_entropy_fused": (_i, [_p, _p, _p, _p, _p, _l, _l, _i, _p], True),
    "mg_matmul": (_i, [_p, _p, _p] + [_l] * 10 + [_i, _p], True),
    "mg_matmul_bt": (_i, [_p, _p, _p] + [_l] * 10 + [_i, _p], True),
    "mg_matmul_bias_bt": (_i, [_p, _p, _p, _p] + [_l] * 10 + [_i, _p], True),
    "mg_linear_bwd": (_i, [_p, _p, _p, _p, _p, _p, _l, _l, _l, _i, _p], True),
    "mg_matmul_bt_add": (_i, [_p, _p, _p, _p, _l, _l, _l, _l, _l, _l, _l, _l, _l, _l, _i, _p], True),
    "mg_matmul_bias_relu_bt": (_i, [_p, _p, _p, _p, _l, _l, _l, _l, _l, _l, _l, _l, _l, _l, _i, _p], True),
    "mg_linear_bwd_fused": (_i, [_p, _p, _p, _p, _p, _p, _l, _l, _l, _i, _i, _i, _p], True),
    "mg_sum_axis": (_i, [_p, _p, _l, _l, _l, _i, _p], True),
    "mg_relu_grad": (_i, [_p, _p, _p, _l, _i, _p], True),
    "mg_softmax": (_i, [_p, _p, _l, _l, _i, _p], True),
    "mg_softmax_grad": (_i, [_p, _p, _p, _l, _l, _i, _p], True),
    "mg_argmax_axis": (_i, [_p, _p, _l, _l, _l, _i, _p], True),
    "mg_adam_step": (_i, [_p, _p, _p, _p, _l, _f, _f, _f, _f, _f, _l, _i, _p], True),
    "mg_sgd_step": (_i, [_p, _p, _l, _f, _p], True),
    "mg_add": (_i, [_p, _p, _p, _l, _i, _p], True),
    "mg_relu": (_i, [_p, _p, _l, _i, _p], True),
    "mg_cast": (_i, [_p, _p, _l, _i, _i, _p], True),
    "mg_contiguous": (_i, [_p, _p, _i, _pl, _pl, _i, _p], True),
    "mg_add_strided": (_i, [_p, _p, _p, _i, _pl, _pl, _pl, _i, _p], True),
    "mg_relu_strided": (_i, [_p, _p, _i, _pl, _pl, _i, _p], True),
    "mg_relu_grad_strided": (_i, [_p, _p, _p, _i, _pl, _pl, _pl, _i, _p], True),
    "mg_cast_strided": (_i, [_p, _p, _i, _pl, _pl, _i, _i, _p], True),
    "mg_softmax_strided": (_i, [_p, _p, _i, _pl, _pl, _i, _p], True),
    "mg_gather": (_i, [_p, _p, _p, _l, _l, _l, _l, _l, _i, _i, _p], True),
    "mg_scatter_add": (_i, [_p, _p, _p, _l, _l, _l, _i, _i, _p], True),
    "mg_deferred_create": (_i, [C.POINTER(_p)], True),
    "mg_deferred_destroy": (_i, [_p], True),
    "mg_deferred_pending": (_i, [_p], False),
    "mg_finish_deferred": (_i, [_p, _p], True),
    "mg_linear_bwd_deferred": (_i, [_p, _p, _p, _p, _p, _p, _l, _l, _l, _i, _i, _i, _i, _p, _p], True),
    "mg_layer_norm_bwd_stats_deferred": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _l, _l, _i, _i, _p, _p], True),
    "mg_linear_bwd_layer_norm_bwd": (_i, [_p] * 12 + [_l, _l, _l, _i, _i, _i, _p, _p], True),
    "mg_scatter_add_deferred": (_i, [_p, _p, _p, _l, _l, _l, _i, _i, _i, _p, _p], True),
    "mg_flash_attn_fwd": (_i, [_p, _p, _p, _p, _p, _p, _l, _l, _l, _l, _f, _i, _i, _i, _p], True),
    "mg_flash_attn_bwd": (_i, [_p] * 10 + [_l, _l, _l, _l, _f, _i, _i, _i, _p], True),
    "mg_flash_attn_fwd_bshd": (_i, [_p, _p, _p, _p, _p, _p, _l, _l, _l, _l, _f, _i, _i, _i, _p], True),
    "mg_flash_attn_bwd_bshd": (_i, [_p] * 10 + [_l, _l, _l, _l, _f, _i, _i, _i, _p], True),
    "mg_flash_attn_fwd_packed": (_i, [_p, _p, _p, _p, _l, _l, _l, _l, _f, _i, _i, _i, _p], True),
    "mg_flash_attn_bwd_packed": (_i, [_p] * 6 + [_l, _l, _l, _l, _f, _i, _i, _i, _p], True),
}


class _Lib:
    """Loaded library with checked wrappers: `lib.mg_xxx(...)` raises on failure."""

    def __init__(self, path: Path):
        self.path = path
        self._dll = C.CDLL(str(path), mode=C.RTLD_GLOBAL)
        self._raw = {}
        missing = []
        for name, (restype, argtypes, _) in PROTOTYPES.items():
            try:
                fn = getattr(self._dll, name)
            except AttributeError:
                missing.append(name)
                continue
            fn.restype = restype
            fn.argtypes = argtypes
            self._raw[name] = fn
        self.missing = missing

    def raw(self, name: str):
        return self._raw[name]

    def has(self, name: str) -> bool:
        return name in self._raw

    def last_error(self) -> str:
        return self._raw["mg_last_error"]().decode("utf-8", "replace")

    def __getattr__(self, name: str):
        if name.startswith("_") or name not in PROTOTYPES:
            raise AttributeError(name)
        if name not in self._raw:
            raise MogradError(2, f"{name} is not exported by {self.path}")
        fn = self._raw[name]
        if not PROTOTYPES[name][2]:
            return fn

        def checked(*args):
            status = fn(*args)
            if status != 0:
                raise MogradError(status, self.last_error())
            return status

        checked.__name__ = name
        setattr(self, name, checked)
        return checked


_LIB: _Lib | None = None


def library_path() -> Path:
    """$MOGRAD_HIP_SO if set, else the in-tree build next to this file."""
    env = os.environ.get("MOGRAD_HIP_SO")
    return Path(env) if env else PKG / LIB_NAME


def load() -> _Lib:
    global _LIB
    if _LIB is None:
        path = library_path()
        if not path.exists():
            raise LibraryMissing(
                f"{path} not found: build it with `python -m mograd_amd.build` (needs hipcc); "
                "there is no CPU fallback for the HIP kernels"
            )
        try:
            _LIB = _Lib(path)
        except OSError as e:  # unresolved ROCm runtime, wrong arch, ...
            raise LibraryMissing(f"cannot load {path}: {e}") from e
    return _LIB
