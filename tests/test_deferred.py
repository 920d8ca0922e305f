"""Deferred second-stage reductions (mg_*_deferred + mg_finish_deferred) against the immediate
entry points: the sums run the same code in the same order, so with grad_dtype equal to the
tensors' dtype no bit may differ, and with float32 the result rounded to the tensors' dtype is
the immediate result.  No counterpart in the reference, which evaluates every reduction where
its graph node stands."""
import ctypes as C

import numpy as np
import pytest

from helpers import integers, normal, uniform

pytestmark = pytest.mark.gpu

from mograd_amd import BF16, F16, F32, I32, AnyBuffer, MogradError  # noqa: E402
from mograd_amd.runtime import round_to_dtype  # noqa: E402

P = lambda b: b.data_ptr() if b is not None else None


class _List:
    def __init__(self, device):
        self.lib = device.lib
        self.h = C.c_void_p()
        self.lib.mg_deferred_create(C.byref(self.h))

    def close(self):
        self.lib.mg_deferred_destroy(self.h)


@pytest.fixture
def pending(device):
    q = _List(device)
    yield q
    q.close()


def _rounded(a32, dtype):
    return round_to_dtype(a32, dtype) if dtype != F32 else a32


@pytest.mark.parametrize("dtype", [BF16, F16, F32])
@pytest.mark.parametrize("M,N,K,with_db", [(2048, 384, 384, False), (4096, 1152, 384, False), (2048, 1536, 384, True),
                                           (4096, 384, 1536, False), (4096, 65, 384, False), (300, 40, 24, True),
                                           (1056, 96, 200, True)])
def test_linear_bwd_deferred_matches_immediate(device, pending, dtype, M, N, K, with_db):
    # Shapes that take the common dX + dW launch (its finishing kernel is what is deferred), the
    # padded 65-wide head, and shapes that have no deferrable second stage (computed at once).
    lib, st = device.lib, device.stream
    x = np.maximum(_rounded(normal(71, 0, (M, K)), dtype), 0)
    w = _rounded(normal(71, 1, (N, K), std=0.05), dtype)
    dy = _rounded(normal(71, 2, (M, N), std=0.5), dtype)
    bx, bw, bdy = (AnyBuffer.from_numpy(device, a, dtype) for a in (x, w, dy))
    dx0, dw0 = AnyBuffer.create(dtype, device, M * K), AnyBuffer.create(dtype, device, N * K)
    db0 = AnyBuffer.create(dtype, device, N) if with_db else None
    lib.mg_linear_bwd_fused(P(bdy), P(bx), P(bw), P(dx0), P(dw0), P(db0), M, N, K, 0, 1, dtype, st)
    for grad_dtype in sorted({dtype, F32}):
        dx = AnyBuffer.create(dtype, device, M * K)
        dw = AnyBuffer.create(grad_dtype, device, N * K, fill=7.0)
        db = AnyBuffer.create(grad_dtype, device, N, fill=7.0) if with_db else None
        lib.mg_linear_bwd_deferred(P(bdy), P(bx), P(bw), P(dx), P(dw), P(db), M, N, K, 0, 1, dtype, grad_dtype, pending.h, st)
        np.testing.assert_array_equal(dx.to_numpy(), dx0.to_numpy(), err_msg="dx is complete before the finish")
        lib.mg_finish_deferred(pending.h, st)
        assert lib.mg_deferred_pending(pending.h) == 0
        got_dw, got_db = dw.to_numpy(), (db.to_numpy() if with_db else None)
        if grad_dtype != dtype:  # fp32 sums: rounding them is what the immediate form stores
            got_dw = round_to_dtype(got_dw, dtype)
            got_db = round_to_dtype(got_db, dtype) if with_db else None
        np.testing.assert_array_equal(got_dw, dw0.to_numpy(), err_msg=f"dw, grad_dtype {grad_dtype}")
        if with_db:
            np.testing.assert_array_equal(got_db, db0.to_numpy(), err_msg=f"db, grad_dtype {grad_dtype}")


@pytest.mark.parametrize("dtype", [BF16, F32])
@pytest.mark.parametrize("rows,cols,residual", [(16384, 384, True), (2048, 4096, False), (64, 384, True), (9, 1000, True),
                                                (3, 40000, False)])
def test_layer_norm_bwd_deferred_matches_immediate(device, pending, dtype, rows, cols, residual):
    lib, st = device.lib, device.stream
    x = _rounded(normal(72, 0, (rows, cols)), dtype)
    g = _rounded(uniform(72, 1, (cols,), 0.5, 1.5), dtype)
    b = _rounded(normal(72, 2, (cols,)), dtype)
    dy = _rounded(normal(72, 3, (rows, cols)), dtype)
    res = _rounded(normal(72, 4, (rows, cols)), dtype)
    bx, bg, bb, bdy, bres = (AnyBuffer.from_numpy(device, a, dtype) for a in (x, g, b, dy, res))
    n = rows * cols
    y, mean, rstd = AnyBuffer.create(dtype, device, n), AnyBuffer.create(F32, device, rows), AnyBuffer.create(F32, device, rows)
    lib.mg_layer_norm_fwd_stats(P(bx), P(bg), P(bb), P(y), P(mean), P(rstd), rows, cols, 1e-5, dtype, st)
    dx0, dg0, db0 = (AnyBuffer.create(dtype, device, m) for m in (n, cols, cols))
    if residual:
        lib.mg_layer_norm_bwd_stats_add(P(bdy), P(bx), P(bg), P(mean), P(rstd), P(bres), P(dx0), P(dg0), P(db0), rows, cols,
                                        dtype, st)
    else:
        lib.mg_layer_norm_bwd_stats(P(bdy), P(bx), P(bg), P(mean), P(rstd), P(dx0), P(dg0), P(db0), rows, cols, dtype, st)
    for grad_dtype in sorted({dtype, F32}):
        dx = AnyBuffer.create(dtype, device, n)
        dg, db = (AnyBuffer.create(grad_dtype, device, cols, fill=7.0) for _ in range(2))
        lib.mg_layer_norm_bwd_stats_deferred(P(bdy), P(bx), P(bg), P(mean), P(rstd), P(bres) if residual else None, P(dx),
                                             P(dg), P(db), rows, cols, dtype, grad_dtype, pending.h, st)
        lib.mg_finish_deferred(pending.h, st)
        np.testing.assert_array_equal(dx.to_numpy(), dx0.to_numpy())
        got_g, got_b = dg.to_numpy(), db.to_numpy()
        if grad_dtype != dtype:
            got_g, got_b = round_to_dtype(got_g, dtype), round_to_dtype(got_b, dtype)
        np.testing.assert_array_equal(got_g, dg0.to_numpy(), err_msg=f"dgamma, grad_dtype {grad_dtype}")
        np.testing.assert_array_equal(got_b, db0.to_numpy(), err_msg=f"dbeta, grad_dtype {grad_dtype}")


@pytest.mark.parametrize("dtype", [BF16, F32])
@pytest.mark.parametrize("n_idx,num_rows,row_size", [(16384, 65, 384), (300, 7, 40), (8192, 2000, 64)])
def test_scatter_add_deferred_matches_immediate(device, pending, dtype, n_idx, num_rows, row_size):
    lib, st = device.lib, device.stream
    idx = integers(73, 0, (n_idx,), 0, num_rows)
    vals = _rounded(normal(73, 1, (n_idx, row_size)), dtype)
    bi, bv = AnyBuffer.from_numpy(device, idx, I32), AnyBuffer.from_numpy(device, vals, dtype)
    want = AnyBuffer.create(dtype, device, num_rows * row_size)
    lib.mg_scatter_add(P(bi), P(bv), P(want), n_idx, num_rows, row_size, I32, dtype, st)
    for grad_dtype in sorted({dtype, F32}):
        dst = AnyBuffer.create(grad_dtype, device, num_rows * row_size, fill=7.0)
        lib.mg_scatter_add_deferred(P(bi), P(bv), P(dst), n_idx, num_rows, row_size, I32, dtype, grad_dtype, pending.h, st)
        lib.mg_finish_deferred(pending.h, st)
        got = dst.to_numpy()
        if grad_dtype != dtype:
            got = round_to_dtype(got, dtype)
        np.testing.assert_array_equal(got, want.to_numpy())


def test_many_sums_finish_in_one_call_and_lists_are_reusable(device, pending):
    # More pending sums than one launch's table holds (64): the finishing call launches as often
    # as needed; a finished list takes new work; a destroyed list drops its sums and returns the
    # partials to the pool.
    lib, st = device.lib, device.stream
    M, N, K, dtype = 2048, 384, 384, BF16
    x = round_to_dtype(normal(74, 0, (M, K)), dtype)
    w = round_to_dtype(normal(74, 1, (N, K), std=0.05), dtype)
    bx, bw = AnyBuffer.from_numpy(device, x, dtype), AnyBuffer.from_numpy(device, w, dtype)
    dys = [AnyBuffer.from_numpy(device, round_to_dtype(normal(74, 10 + i, (M, N), std=0.5), dtype), dtype) for i in range(3)]
    want = []
    dx = AnyBuffer.create(dtype, device, M * K)
    for bdy in dys:
        dw, db = AnyBuffer.create(dtype, device, N * K), AnyBuffer.create(dtype, device, N)
        lib.mg_linear_bwd(P(bdy), P(bx), P(bw), P(dx), P(dw), P(db), M, N, K, dtype, st)
        want.append((dw.to_numpy(), db.to_numpy()))
    for rounds in range(2):
        outs = []
        for i in range(40):  # 80 sums
            dw, db = AnyBuffer.create(dtype, device, N * K, fill=3.0), AnyBuffer.create(dtype, device, N, fill=3.0)
            lib.mg_linear_bwd_deferred(P(dys[i % 3]), P(bx), P(bw), P(dx), P(dw), P(db), M, N, K, 0, 0, dtype, dtype,
                                       pending.h, st)
            outs.append((dw, db))
        assert lib.mg_deferred_pending(pending.h) == 80
        lib.mg_finish_deferred(pending.h, st)
        for i, (dw, db) in enumerate(outs):
            np.testing.assert_array_equal(dw.to_numpy(), want[i % 3][0], err_msg=f"dw {i}")
            np.testing.assert_array_equal(db.to_numpy(), want[i % 3][1], err_msg=f"db {i}")
    other = _List(device)
    dw, db = AnyBuffer.create(dtype, device, N * K, fill=3.0), AnyBuffer.create(dtype, device, N)
    lib.mg_linear_bwd_deferred(P(dys[0]), P(bx), P(bw), P(dx), P(dw), P(db), M, N, K, 0, 0, dtype, dtype, other.h, st)
    held = device.memory_stats().allocated_bytes
    other.close()
    assert device.memory_stats().allocated_bytes < held, "destroying a list returns its partials to the pool"
    device.synchronize()
    assert np.all(dw.to_numpy() == 3.0), "a dropped sum writes nothing"


def test_deferred_errors(device, pending):
    lib, st = device.lib, device.stream
    a = AnyBuffer.create(BF16, device, 64 * 64)
    with pytest.raises(MogradError, match="null deferred list"):
        lib.mg_linear_bwd_deferred(P(a), P(a), P(a), P(a), P(a), None, 64, 64, 64, 0, 0, BF16, BF16, None, st)
    with pytest.raises(MogradError, match="grad_dtype"):
        lib.mg_linear_bwd_deferred(P(a), P(a), P(a), P(a), P(a), None, 64, 64, 64, 0, 0, BF16, F16, pending.h, st)
    with pytest.raises(MogradError, match="grad_dtype"):
        lib.mg_scatter_add_deferred(P(a), P(a), P(a), 4, 4, 4, I32, F32, BF16, pending.h, st)
    with pytest.raises(MogradError, match="null deferred list"):
        lib.mg_finish_deferred(None, st)
    assert lib.mg_deferred_pending(pending.h) == 0
