"""No-GPU checks of the boundary: the shared library loads, exports every symbol the
header declares, and the host-side layout logic matches the reference's."""
import re
from pathlib import Path

import pytest

import mograd_amd
from mograd_amd import Layout, MogradError, _lib
from oracle import oracle_np as O

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "mograd_hip.h"


def _declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(mg_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = mograd_amd.load()  # raises LibraryMissing if the .so has not been built
    declared = _declared_symbols()
    assert len(declared) >= 40
    import ctypes

    dll = ctypes.CDLL(str(lib.path))
    missing = [name for name in declared if not hasattr(dll, name)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_binding_covers_the_header():
    declared = set(_declared_symbols())
    bound = set(_lib.PROTOTYPES)
    assert declared == bound, f"header-only: {declared - bound}; binding-only: {bound - declared}"


def test_pure_host_entry_points():
    lib = mograd_amd.load()
    assert lib.mg_version().startswith(b"mograd_hip")
    # size classes: mograd/memory.mojo:59-72, tests/test_memory.mojo:18-30
    assert lib.mg_round_class(1000) == 1024 and lib.mg_round_class(1025) == 1152
    for n in [0, 1, 511, 512, 513, 990, 4096, 5000, 123457, (1 << 20) + 1, 3 << 30]:
        assert lib.mg_round_class(n) == O.round_class(n)
    assert lib.mg_pool_enabled() in (0, 1)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setenv("MOGRAD_HIP_SO", str(tmp_path / "nope.so"))
    monkeypatch.setattr(_lib, "_LIB", None)
    with pytest.raises(mograd_amd.LibraryMissing):
        _lib.load()


def test_layout_contiguity_and_views():
    l = Layout(4, 6)
    assert l.is_contiguous() and l.stride() == (6, 1) and l.numel() == 24
    t = l.transpose()
    assert t.shape() == (6, 4) and t.stride() == (1, 6) and not t.is_contiguous()
    assert t.as_contiguous().stride() == (4, 1)
    s = Layout(4, 2).slice_axis(0, 0, 4, 2)
    assert s.shape() == (2, 2) and s.stride() == (4, 1) and not s.is_contiguous()
    assert Layout(4, 2).slice_axis(0, 1, 4, 2).base_offset == 2


def test_layout_batch_dims_collapsible():
    # mograd/layout.mojo:214-236
    assert Layout(2, 3, 4, 5).batch_dims_collapsible()
    assert not Layout(2, 3, 4, 5).transpose(1, 2).batch_dims_collapsible()
    assert Layout(3, 4, 5).transpose(0, 1).batch_dims_collapsible()  # a single batch axis always is
    assert Layout(2, 3, 4, 5, strides=(0, 0, 5, 1)).batch_dims_collapsible()  # all-broadcast batch axes


def test_layout_reduce_dims():
    # mograd/layout.mojo:287-298
    assert Layout(2048, 4096).reduce_dims(0) == (1, 2048, 4096)
    assert Layout(3, 50, 8).reduce_dims(1) == (3, 50, 8)
    assert Layout(4, 6, 10).reduce_dims(-1) == (24, 10, 1)
    with pytest.raises(MogradError):
        Layout(4, 6).reduce_dims(2)


def test_scheduler_rules_cover_the_path():
    from mograd_amd import SCHEDULER_RULES

    assert set(SCHEDULER_RULES) == {
        "ADD", "RELU", "CAST", "CONTIGUOUS", "GATHER", "SCATTER_ADD", "RELU_GRAD", "SOFTMAX", "SOFTMAX_GRAD", "ARGMAX", "SUM", "MATMUL", "MATMUL_BT", "MATMUL_BIAS_BT", "LAYER_NORM", "LAYER_NORM_GRAD", "FLASH_ATTN",
        "FLASH_ATTN_GRAD", "CROSS_ENTROPY", "CROSS_ENTROPY_GRAD",
        # fused nodes of the gradient rules the reference lacks
        "LINEAR_GRAD", "LAYER_NORM_STATS", "LAYER_NORM_STATS_GRAD", "CROSS_ENTROPY_IDS", "CROSS_ENTROPY_IDS_GRAD",
        # views, and the fused nodes of mograd_amd.rewrites.GPU_REWRITES
        "RESHAPE", "TRANSPOSE", "EXPAND", "MATMUL_BT_ADD", "MATMUL_BIAS_RELU_BT", "LAYER_NORM_STATS_GRAD_ADD", "LINEAR_LAYER_NORM_GRAD",
        "FLASH_ATTN_PACKED",
        "FLASH_ATTN_PACKED_GRAD"}
