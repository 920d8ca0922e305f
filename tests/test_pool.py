"""The caching pool on the GPU, following the reference's tests/test_memory.mojo."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from mograd_amd import F32, AnyBuffer, Layout  # noqa: E402
from mograd_amd import runtime as R  # noqa: E402

U8 = None  # bytes are requested through the raw pool calls


def _alloc(device, nbytes):
    p = C.c_void_p()
    device.lib.mg_pool_alloc(C.byref(p), nbytes)
    return p.value


def _free(device, ptr):
    device.lib.mg_pool_free(C.c_void_p(ptr))


def test_size_classes_round_up(device):
    # tests/test_memory.mojo:18-30
    if not device.pool_enabled():
        pytest.skip("MOGRAD_POOL=0")
    p1000 = _alloc(device, 1000)
    _free(device, p1000)
    p1024 = _alloc(device, 1024)
    assert p1024 == p1000
    p1025 = _alloc(device, 1025)
    assert p1025 != p1000
    _free(device, p1024)
    _free(device, p1025)


def test_reuse_and_class_sharing(device):
    # tests/test_memory.mojo:44-60
    if not device.pool_enabled():
        pytest.skip("MOGRAD_POOL=0")
    b = AnyBuffer.create(F32, device, 1000)
    p1 = b.data_ptr().value
    del b
    b2 = AnyBuffer.create(F32, device, 1000)
    assert b2.data_ptr().value == p1
    del b2
    p = _alloc(device, 1000)
    _free(device, p)
    q = _alloc(device, 990)  # same 1024-byte class
    assert q == p
    _free(device, q)


def test_view_keeps_storage_alive(device):
    # tests/test_memory.mojo:63-92
    if not device.pool_enabled():
        pytest.skip("MOGRAD_POOL=0")
    b = AnyBuffer.create(F32, device, 256)
    v = b.view(Layout(16, 16))
    p1 = v.data_ptr().value
    del b
    other = AnyBuffer.create(F32, device, 256)
    assert other.data_ptr().value != p1  # the view still co-owns the block
    del v
    reused = AnyBuffer.create(F32, device, 256)
    assert reused.data_ptr().value == p1
    assert other.data_ptr().value != reused.data_ptr().value


def test_empty_cache_drops_reserved(device):
    # tests/test_memory.mojo:110-124
    if not device.pool_enabled():
        pytest.skip("MOGRAD_POOL=0")
    b = AnyBuffer.create(F32, device, 4096)
    del b
    st = device.memory_stats()
    assert st.reserved_bytes > st.allocated_bytes
    device.synchronize()
    device.empty_cache()
    st = device.memory_stats()
    assert st.reserved_bytes == st.allocated_bytes
    misses = st.miss_count
    b = AnyBuffer.create(F32, device, 4096)
    assert device.memory_stats().miss_count == misses + 1


def test_stats_counts(device):
    # tests/test_memory.mojo:133-150
    if not device.pool_enabled():
        pytest.skip("MOGRAD_POOL=0")
    device.synchronize()
    device.empty_cache()
    t0 = device.memory_stats()
    b1 = AnyBuffer.create(F32, device, 1024)
    b2 = AnyBuffer.create(F32, device, 1024)
    assert b1.data_ptr().value != b2.data_ptr().value
    del b1, b2
    st = device.memory_stats()
    assert st.miss_count == t0.miss_count + 2
    assert st.free_count == t0.free_count + 2
    assert st.allocated_bytes == t0.allocated_bytes
    assert st.peak_allocated >= t0.allocated_bytes + 8192
    assert st.reserved_bytes >= 8192
    b3 = AnyBuffer.create(F32, device, 1024)
    st = device.memory_stats()
    assert st.hit_count == t0.hit_count + 1
    assert st.allocated_bytes == t0.allocated_bytes + 4096
    assert b3.data_ptr().value != 0
    assert "mograd memory pool:" in device.memory_summary()


def test_kernel_scratch_returns_to_the_pool(device):
    # LayerNorm backward takes two scratch buffers and hands them back before returning
    rows, cols = 64, 256
    x = AnyBuffer.from_numpy(device, np.ones((rows, cols), np.float32))
    g = AnyBuffer.from_numpy(device, np.ones(cols, np.float32))
    dx, dg, db = (AnyBuffer.create(F32, device, n) for n in (rows * cols, cols, cols))
    before = device.memory_stats().allocated_bytes
    device.lib.mg_layer_norm_bwd(x.data_ptr(), x.data_ptr(), g.data_ptr(), dx.data_ptr(), dg.data_ptr(),
                                 db.data_ptr(), rows, cols, 1e-5, F32, device.stream)
    assert device.memory_stats().allocated_bytes == before
    device.synchronize()


def test_free_of_foreign_pointer_is_an_error(device):
    with pytest.raises(R.MogradError, match="not allocated by this pool"):
        device.lib.mg_pool_free(C.c_void_p(0x1000))
