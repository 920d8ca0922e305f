"""Softmax cross-entropy forward / gradient / fused on the GPU against the float64 oracle.

Mirrors the reference's tests (tests/test_ops.mojo:155-186,
tests/test_non_contiguous.mojo:275-310, tests/test_grad.mojo:432-483) through the same
dispatch surface, then random shapes that reach every kernel, the integer-label and
fused entry points, and the benchmark shape.
"""
import ctypes as C

import numpy as np
import pytest

from helpers import ATOL_F32, RTOL_F32, assert_close, golden, integers, normal
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu

from mograd_amd import BF16, F16, F32, I32, I64, AnyBuffer, Layout, MogradError, Node  # noqa: E402
from mograd_amd import runtime as R  # noqa: E402
from mograd_amd.runtime import round_to_dtype  # noqa: E402


def _ce(device, logits, labels, la=None, lb=None, dtype=F32):
    """CROSS_ENTROPY through the dispatch surface.  la/lb are the operand layouts (views
    over the uploaded arrays); default contiguous."""
    logits, labels = np.asarray(logits, np.float32), np.asarray(labels, np.float32)
    la = la or Layout(*logits.shape)
    lb = lb or Layout(*labels.shape)
    node = Node("CROSS_ENTROPY", Layout(1), dtype, [Node.leaf(la, dtype), Node.leaf(lb, dtype)])
    bl, by = AnyBuffer.from_numpy(device, logits, dtype), AnyBuffer.from_numpy(device, labels, dtype)
    (out,) = R.run(node, [bl.view(la), by.view(lb)], device)
    return out.item()


def _ce_grad(device, logits, labels, upstream=1.0, la=None, lb=None, dtype=F32):
    logits, labels = np.asarray(logits, np.float32), np.asarray(labels, np.float32)
    la = la or Layout(*logits.shape)
    lb = lb or Layout(*labels.shape)
    node = Node("CROSS_ENTROPY_GRAD", la.as_contiguous(), dtype,
                [Node.leaf(la, dtype), Node.leaf(lb, dtype), Node.leaf(Layout(1), dtype)])
    bl, by = AnyBuffer.from_numpy(device, logits, dtype), AnyBuffer.from_numpy(device, labels, dtype)
    bu = AnyBuffer.from_numpy(device, np.array([upstream], np.float32), dtype)
    (out,) = R.run(node, [bl.view(la), by.view(lb), bu], device)
    return out.to_numpy(la.shape())


# ---- the reference's golden values -----------------------------------------------


@pytest.mark.parametrize("g", golden("cross_entropy"), ids=lambda g: g["cite"])
def test_goldens_contiguous(device, g):
    assert abs(_ce(device, g["logits"], g["labels"]) - g["loss"]) < g["atol"]


def test_goldens_strided(device):
    # tests/test_non_contiguous.mojo:275-299
    logits = np.array([[0, 0], [100, 0], [0, 0], [0, 0]], np.float32)
    sl = Layout(4, 2).slice_axis(0, 0, 4, 2)
    assert not sl.is_contiguous()
    assert abs(_ce(device, logits, np.full((2, 2), 0.5), la=sl) - 0.693147) < 1e-3
    labels_full = np.array([[1, 0], [99, 99], [0, 1], [99, 99]], np.float32)
    assert abs(_ce(device, np.zeros((2, 2)), labels_full, lb=sl) - 0.693147) < 1e-3
    t = Layout(2, 2).transpose()
    assert not t.is_contiguous()
    assert abs(_ce(device, np.zeros((2, 2)), np.eye(2), lb=t) - 0.693147) < 1e-3


@pytest.mark.parametrize("g", golden("cross_entropy_grad"), ids=lambda g: g["cite"])
def test_grad_golden_transposed_logits(device, g):
    # The logits operand is the transposed view of `a`; the gradient arrives in the layout of
    # that view, and the expected numbers are for the underlying array a.
    a = np.array(g["a"], np.float32)
    d = _ce_grad(device, a, g["labels"], g["upstream"], la=Layout(*a.shape).transpose())
    np.testing.assert_allclose(d.T.reshape(-1), g["grad_a_flat"], atol=g["atol"])


def test_grad_rows_sum_to_zero_and_rank3(device):
    d = _ce_grad(device, np.ones((4, 10)), O.one_hot([0, 1, 2, 3], 10))
    assert np.max(np.abs(d.sum(axis=1))) < 1e-4
    x = (np.arange(24) * 0.1).reshape(2, 3, 4).astype(np.float32)
    y = O.one_hot([0, 2, 1, 3, 0, 1], 4).reshape(2, 3, 4)
    assert abs(_ce(device, x, y) - _ce(device, x.reshape(6, 4), y.reshape(6, 4))) < 1e-4
    np.testing.assert_allclose(_ce_grad(device, x, y).reshape(6, 4),
                               _ce_grad(device, x.reshape(6, 4), y.reshape(6, 4)), atol=1e-4)


# ---- random shapes: every register layout, scalar path, streaming fallback ----------

SHAPES = [(1, 1), (4, 3), (64, 10), (37, 65), (5, 256), (9, 1000), (6, 4096), (3, 8192), (7, 10007), (5, 32768),
          (3, 50304), (4, 65536), (2, 70000), (2, 100003), (300, 130)]


@pytest.mark.parametrize("N,Cc", SHAPES)
def test_dense_random_f32(device, N, Cc):
    x = normal(30, 0, (N, Cc), std=2.0)
    soft = np.abs(normal(30, 1, (N, Cc))) + 0.01
    soft = (soft / soft.sum(axis=1, keepdims=True)).astype(np.float32)
    assert_close(_ce(device, x, soft), O.cross_entropy(x, soft), RTOL_F32, ATOL_F32, "loss")
    # gradient entries are (p - y) * upstream / N: compare at the parity rtol with an
    # absolute floor at the same relative level of that natural scale
    want = O.cross_entropy_grad(x, soft, 0.75)
    assert_close(_ce_grad(device, x, soft, 0.75), want, RTOL_F32, RTOL_F32 * 0.75 / N, "dlogits")


def _ids_calls(device, x, ids, upstream, id_dtype, dtype=F32):
    N, Cc = x.shape
    lib = device.lib
    bx = AnyBuffer.from_numpy(device, x, dtype)
    bi = AnyBuffer.from_numpy(device, ids.astype(np.int64 if id_dtype == I64 else np.int32), id_dtype)
    bu = AnyBuffer.from_numpy(device, np.array([upstream], np.float32), dtype)
    loss = AnyBuffer.create(dtype, device, 1)
    lib.mg_cross_entropy_ids(bx.data_ptr(), bi.data_ptr(), loss.data_ptr(), N, Cc, dtype, id_dtype, device.stream)
    grad = AnyBuffer.create(dtype, device, N * Cc)
    lib.mg_cross_entropy_grad_ids(bx.data_ptr(), bi.data_ptr(), bu.data_ptr(), grad.data_ptr(), N, Cc, dtype,
                                  id_dtype, device.stream)
    loss2 = AnyBuffer.create(dtype, device, 1)
    grad2 = AnyBuffer.create(dtype, device, N * Cc)
    lib.mg_cross_entropy_fused_ids(bx.data_ptr(), bi.data_ptr(), bu.data_ptr(), loss2.data_ptr(), grad2.data_ptr(),
                                   N, Cc, dtype, id_dtype, device.stream)
    return loss.item(), grad.to_numpy((N, Cc)), loss2.item(), grad2.to_numpy((N, Cc))


@pytest.mark.parametrize("id_dtype", [I32, I64])
@pytest.mark.parametrize("N,Cc", SHAPES)
def test_ids_random_f32(device, N, Cc, id_dtype):
    x = normal(31, 0, (N, Cc), std=2.0)
    ids = integers(31, 1, (N,), 0, Cc)
    loss, grad, loss2, grad2 = _ids_calls(device, x, ids, 1.25, id_dtype)
    want_loss = O.cross_entropy_ids(x, ids)
    want = O.cross_entropy_grad_ids(x, ids, 1.25)
    assert_close(loss, want_loss, RTOL_F32, ATOL_F32, "loss")
    assert_close(loss2, want_loss, RTOL_F32, ATOL_F32, "fused loss")
    floor = RTOL_F32 * 1.25 / N
    assert_close(grad, want, RTOL_F32, floor, "dlogits")
    np.testing.assert_array_equal(grad, grad2)  # the fused call runs the same gradient code
    # label gather is exact: the only negative entries of the gradient sit at the labels
    if Cc > 1:
        neg_cols = [np.flatnonzero(grad[r] < 0) for r in range(N)]
        assert all(list(c) == [ids[r]] for r, c in enumerate(neg_cols))
    # ids equal the dense one-hot form
    one_hot = O.one_hot(ids, Cc).astype(np.float32)
    assert_close(_ce(device, x, one_hot), want_loss, RTOL_F32, ATOL_F32, "dense loss")
    assert_close(_ce_grad(device, x, one_hot, 1.25), want, RTOL_F32, floor, "dense dlogits")


def test_fused_dense(device):
    N, Cc = 33, 5000
    x = normal(32, 0, (N, Cc), std=2.0)
    soft = np.abs(normal(32, 1, (N, Cc))) + 0.01
    soft = (soft / soft.sum(axis=1, keepdims=True)).astype(np.float32)
    bx, by = AnyBuffer.from_numpy(device, x), AnyBuffer.from_numpy(device, soft)
    bu = AnyBuffer.from_numpy(device, np.array([0.5], np.float32))
    loss, grad = AnyBuffer.create(F32, device, 1), AnyBuffer.create(F32, device, N * Cc)
    device.lib.mg_cross_entropy_fused(bx.data_ptr(), by.data_ptr(), bu.data_ptr(), loss.data_ptr(), grad.data_ptr(),
                                      N, Cc, F32, device.stream)
    assert_close(loss.item(), O.cross_entropy(x, soft), RTOL_F32, ATOL_F32, "loss")
    want = O.cross_entropy_grad(x, soft, 0.5)
    assert_close(grad.to_numpy((N, Cc)), want, RTOL_F32, RTOL_F32 * 0.5 / N, "dlogits")


def test_benchmark_shape_rows(device):
    # fp32 logits (8192, 50304) ~ N(0, 2), int32 labels: checked on a 512-row slab against
    # the oracle (the oracle needs seconds per 1000 rows), with the row count of the full
    # problem folded into the upstream scale; then full size through properties.
    N, Cc = 512, 50304
    x = normal(2, 10, (N, Cc), std=2.0)
    ids = integers(2, 11, (N,), 0, Cc)
    loss, grad, loss2, grad2 = _ids_calls(device, x, ids, 1.0, I32)
    assert_close(loss2, O.cross_entropy_ids(x, ids), RTOL_F32, ATOL_F32, "loss")
    want = O.cross_entropy_grad_ids(x, ids)
    assert_close(grad2, want, RTOL_F32, RTOL_F32 / N, "dlogits")


def test_benchmark_shape_full_properties(device):
    N, Cc = 8192, 50304
    lib = device.lib
    rng = np.random.Generator(np.random.PCG64(2012))
    grad = AnyBuffer.create(F32, device, N * Cc)
    logits = AnyBuffer.create(F32, device, N * Cc)
    ids = integers(2, 13, (N,), 0, Cc)
    # Upload in slabs to bound host memory; the oracle's loss is accumulated per slab.
    slab = 1024
    want_loss = 0.0
    for r0 in range(0, N, slab):
        part = (rng.standard_normal((slab, Cc), dtype=np.float32) * 2.0)
        want_loss += O.cross_entropy_ids(part, ids[r0:r0 + slab]) * slab / N
        lib.mg_copy_to_device(C.c_void_p(logits.data_ptr().value + r0 * Cc * 4), part.ctypes.data_as(C.c_void_p),
                              part.nbytes, device.stream)
    bi = AnyBuffer.from_numpy(device, ids, I32)
    loss = AnyBuffer.create(F32, device, 1)
    lib.mg_cross_entropy_fused_ids(logits.data_ptr(), bi.data_ptr(), None, loss.data_ptr(), grad.data_ptr(), N, Cc,
                                   F32, I32, device.stream)
    assert_close(loss.item(), want_loss, RTOL_F32, ATOL_F32, "loss")
    g = grad.to_numpy((N, Cc))
    # every row of dlogits sums to zero; exactly one negative entry per row, at the label
    assert np.max(np.abs(g.astype(np.float64).sum(axis=1))) < 1e-8
    neg = g < 0
    assert np.all(neg.sum(axis=1) == 1)
    assert np.array_equal(np.argmax(neg, axis=1), ids)
    # loss-only entry agrees with the oracle too
    loss_only = AnyBuffer.create(F32, device, 1)
    lib.mg_cross_entropy_ids(logits.data_ptr(), bi.data_ptr(), loss_only.data_ptr(), N, Cc, F32, I32, device.stream)
    assert_close(loss_only.item(), want_loss, RTOL_F32, ATOL_F32, "loss-only")


@pytest.mark.parametrize("dtype,rtol", [(F16, 2e-3), (BF16, 1.6e-2)])
@pytest.mark.parametrize("N,Cc", [(64, 65), (9, 1000), (5, 50304), (3, 140000)])
def test_half_precision_storage(device, dtype, rtol, N, Cc):
    x = round_to_dtype(normal(33, 0, (N, Cc), std=2.0), dtype)
    ids = integers(33, 1, (N,), 0, Cc)
    one_hot = O.one_hot(ids, Cc).astype(np.float32)
    up = float(round_to_dtype(np.array([1.5], np.float32), dtype)[0])
    loss, grad, loss2, grad2 = _ids_calls(device, x, ids, up, I64, dtype)
    want_loss = O.cross_entropy_ids(x, ids)
    want = O.cross_entropy_grad_ids(x, ids, up)
    floor = rtol * up / N
    assert_close(loss, want_loss, rtol, rtol, "loss")
    assert_close(loss2, want_loss, rtol, rtol, "fused loss")
    assert_close(grad, want, rtol, floor, "dlogits")
    assert_close(_ce(device, x, one_hot, dtype=dtype), want_loss, rtol, rtol, "dense loss")
    assert_close(_ce_grad(device, x, one_hot, up, dtype=dtype), want, rtol, floor, "dense dlogits")


@pytest.mark.parametrize("dtype,rtol", [(F16, 2e-3), (BF16, 1.6e-2)])
@pytest.mark.parametrize("N,Cc", [(5, 50304), (3, 40008), (2, 70000), (2, 110000), (3, 32776), (9, 4104), (7, 12000),
                                  (4, 24000), (6, 8192)])
def test_wide_16bit_rows_stay_packed(device, monkeypatch, dtype, rtol, N, Cc):
    # 16-bit rows of 4104 to 131072 columns with integer labels stay in registers as loaded
    # and are unpacked once per pass (256, 512 or 1024 threads per row); MOGRAD_HIP_CE_PACKED=0
    # holds them as fp32.  The arithmetic per element is the same: same bits; both meet the oracle.
    x = round_to_dtype(normal(35, 0, (N, Cc), std=2.0), dtype)
    ids = integers(35, 1, (N,), 0, Cc)
    ids[0] = Cc - 1  # a label in the row's last, possibly partial, chunk
    got = {}
    for knob in ("1", "0"):
        monkeypatch.setenv("MOGRAD_HIP_CE_PACKED", knob)
        got[knob] = _ids_calls(device, x, ids, 1.0, I32, dtype)
    want_loss, want = O.cross_entropy_ids(x, ids), O.cross_entropy_grad_ids(x, ids, 1.0)
    for knob, (loss, grad, loss2, grad2) in got.items():
        assert_close(loss2, want_loss, rtol, rtol, f"fused loss ({knob})")
        assert_close(grad, want, rtol, rtol / N, f"dlogits ({knob})")
        assert_close(grad2, want, rtol, rtol / N, f"fused dlogits ({knob})")
    np.testing.assert_array_equal(got["1"][1], got["0"][1])
    np.testing.assert_array_equal(got["1"][3], got["0"][3])
    assert got["1"][2] == got["0"][2]


def test_out_of_range_id_flags_loss(device):
    x = normal(34, 0, (4, 100))
    ids = np.array([0, 5, 100, 7], np.int32)
    loss, grad, loss2, _ = _ids_calls(device, x, ids, 1.0, I32)
    assert np.isnan(loss) and np.isnan(loss2)
    assert np.all(np.isfinite(grad))  # the row's gradient is plain softmax / N; nothing is read out of bounds


def test_errors(device):
    buf = AnyBuffer.create(F32, device, 16)
    p = buf.data_ptr()
    with pytest.raises(MogradError, match="unsupported dtype"):
        device.lib.mg_cross_entropy(p, p, p, 2, 4, I64, device.stream)
    with pytest.raises(MogradError, match="bad shape"):
        device.lib.mg_cross_entropy(p, p, p, 0, 4, F32, device.stream)
    with pytest.raises(MogradError, match="ids must be int32 or int64"):
        device.lib.mg_cross_entropy_ids(p, p, p, 2, 4, F32, F32, device.stream)
    with pytest.raises(MogradError, match="rank"):
        shape = (C.c_int64 * 9)(*([1] * 9))
        device.lib.mg_cross_entropy_strided(p, p, p, 9, shape, shape, shape, F32, device.stream)
