"""The entry point that allocates nothing: mg_cross_entropy_fused_ids_noalloc keeps its
per-row loss terms in a static device array instead of a pool block.  Checked against
mg_cross_entropy_fused_ids (bit for bit: same kernels, same order of sums) on two calls
in a row, the second with a smaller input, and against the float64 oracle."""
import numpy as np
import pytest

from helpers import ATOL_F32, RTOL_F32, assert_close, integers, normal
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu

from mograd_amd import BF16, F32, I32, I64, AnyBuffer, MogradError  # noqa: E402
from mograd_amd._lib import PoolStats  # noqa: E402
from mograd_amd.runtime import round_to_dtype  # noqa: E402


def _both(device, logits, ids, dtype, id_dtype):
    lib, st = device.lib, device.stream
    n, c = logits.shape
    bl = AnyBuffer.from_numpy(device, logits, dtype)
    bi = AnyBuffer.from_numpy(device, ids, id_dtype)
    out = []
    for name in ("mg_cross_entropy_fused_ids", "mg_cross_entropy_fused_ids_noalloc"):
        loss = AnyBuffer.create(dtype, device, 1, fill=7.0)
        grad = AnyBuffer.create(dtype, device, n * c, fill=7.0)
        before, after = PoolStats(), PoolStats()
        lib.mg_pool_get_stats(before)
        getattr(lib, name)(bl.data_ptr(), bi.data_ptr(), None, loss.data_ptr(), grad.data_ptr(), n, c, dtype, id_dtype, st)
        lib.mg_pool_get_stats(after)
        out.append((loss.to_numpy(), grad.to_numpy((n, c)), (after.hit_count + after.miss_count) - (before.hit_count + before.miss_count)))
    return out


@pytest.mark.parametrize("dtype,id_dtype,np_id", [(F32, I32, np.int32), (BF16, I64, np.int64)])
def test_noalloc_equals_the_pool_form_on_two_calls(device, dtype, id_dtype, np_id):
    # first call large, second smaller: the static array still holds the first call's terms
    for cfg, (n, c) in enumerate([(3000, 1000), (517, 333)]):
        logits = round_to_dtype(normal(70, cfg, (n, c), std=2.0), dtype)
        ids = integers(70, 10 + cfg, (n,), 0, c, np_id)
        (loss_a, grad_a, allocs_a), (loss_b, grad_b, allocs_b) = _both(device, logits, ids, dtype, id_dtype)
        assert allocs_a == 1 and allocs_b == 0, "the non-allocating form must take nothing from the pool"
        np.testing.assert_array_equal(loss_b, loss_a)
        np.testing.assert_array_equal(grad_b, grad_a)
        if dtype == F32:
            assert_close(loss_b[0], O.cross_entropy_ids(logits, ids), RTOL_F32, ATOL_F32, "loss")
            assert_close(grad_b, O.cross_entropy_grad_ids(logits, ids), RTOL_F32, ATOL_F32 / n, "dlogits")


def test_noalloc_rejects_more_rows_than_the_static_array(device):
    buf = AnyBuffer.create(F32, device, 64)
    p = buf.data_ptr()
    with pytest.raises(MogradError, match=r"exceeds the 1048576 rows of the static scratch"):
        device.lib.mg_cross_entropy_fused_ids_noalloc(p, p, None, p, p, (1 << 20) + 1, 4, F32, I32, device.stream)


def test_noalloc_call_replays_from_a_hip_graph(device):
    # What the entry point exists for: a caller that records its work into a HIP graph, where no
    # allocation may happen.  One call is captured (after mg_init has resolved the static array, so
    # the capture sees kernel launches only: no memset or copy nodes), the graph is replayed three
    # times with eager calls on other inputs and synchronisations in between (they overwrite the
    # static array, which every replay must refill for itself), and every replay must give the
    # bits of the eager call.
    import ctypes as C

    hip = C.CDLL("libamdhip64.so")
    lib, st = device.lib, device.stream
    n, c = 2048, 777
    logits = normal(71, 0, (n, c), std=2.0)
    ids = integers(71, 1, (n,), 0, c, np.int32)
    other_logits = normal(71, 2, (n + 100, c), std=2.0)
    other_ids = integers(71, 3, (n + 100,), 0, c, np.int32)
    bl, bi = AnyBuffer.from_numpy(device, logits, F32), AnyBuffer.from_numpy(device, ids, I32)
    bol, boi = AnyBuffer.from_numpy(device, other_logits, F32), AnyBuffer.from_numpy(device, other_ids, I32)
    loss_e, grad_e = AnyBuffer.create(F32, device, 1), AnyBuffer.create(F32, device, n * c)
    lib.mg_cross_entropy_fused_ids_noalloc(bl.data_ptr(), bi.data_ptr(), None, loss_e.data_ptr(), grad_e.data_ptr(), n, c,
                                           F32, I32, st)
    want_loss, want_grad = loss_e.to_numpy(), grad_e.to_numpy()
    loss_g, grad_g = AnyBuffer.create(F32, device, 1), AnyBuffer.create(F32, device, n * c)
    scratch_loss, scratch_grad = AnyBuffer.create(F32, device, 1), AnyBuffer.create(F32, device, (n + 100) * c)
    device.synchronize()

    def ok(rc, what):
        assert rc == 0, f"{what} failed with hipError {rc}"

    graph, graph_exec = C.c_void_p(), C.c_void_p()
    before, after = PoolStats(), PoolStats()
    lib.mg_pool_get_stats(before)
    ok(hip.hipStreamBeginCapture(st, C.c_int(2)), "hipStreamBeginCapture")  # relaxed mode
    try:
        lib.mg_cross_entropy_fused_ids_noalloc(bl.data_ptr(), bi.data_ptr(), None, loss_g.data_ptr(), grad_g.data_ptr(), n,
                                               c, F32, I32, st)
    finally:
        ok(hip.hipStreamEndCapture(st, C.byref(graph)), "hipStreamEndCapture")
    lib.mg_pool_get_stats(after)
    assert (after.hit_count, after.miss_count, after.alloc_count) == (before.hit_count, before.miss_count, before.alloc_count)
    ok(hip.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, C.c_size_t(0)), "hipGraphInstantiate")
    try:
        for replay in range(3):
            lib.mg_fill(loss_g.data_ptr(), 7.0, 1, F32, st)
            lib.mg_fill(grad_g.data_ptr(), 7.0, n * c, F32, st)
            lib.mg_cross_entropy_fused_ids_noalloc(bol.data_ptr(), boi.data_ptr(), None, scratch_loss.data_ptr(),
                                                   scratch_grad.data_ptr(), n + 100, c, F32, I32, st)
            device.synchronize()
            ok(hip.hipGraphLaunch(graph_exec, st), "hipGraphLaunch")
            device.synchronize()
            np.testing.assert_array_equal(loss_g.to_numpy(), want_loss, err_msg=f"loss, replay {replay}")
            np.testing.assert_array_equal(grad_g.to_numpy(), want_grad, err_msg=f"dlogits, replay {replay}")
    finally:
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)
