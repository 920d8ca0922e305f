"""LayerNorm forward/backward on the GPU against the float64 oracle.

Mirrors the reference's LayerNorm tests (tests/test_nn.mojo:283-324,
tests/test_grad.mojo:776-856) through the same dispatch surface, then random shapes that
reach every kernel layout, the benchmark shape, and the edge cases.
"""
import numpy as np
import pytest

from helpers import ATOL_F32, RTOL_F32, assert_close, assert_sum_close, golden, normal, uniform
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu

from mograd_amd import BF16, F16, F32, AnyBuffer, Layout, MogradError, Node  # noqa: E402
from mograd_amd import runtime as R  # noqa: E402
from mograd_amd.runtime import round_to_dtype  # noqa: E402


def _ln_fwd(device, x, gamma, beta, eps=1e-5, dtype=F32):
    shape = np.asarray(x).shape
    node = Node("LAYER_NORM", Layout(*shape), dtype,
                [Node.leaf(Layout(*shape), dtype), Node.leaf(Layout(shape[-1]), dtype), Node.leaf(Layout(shape[-1]), dtype)],
                {"eps": eps, "axis": -1})
    bufs = [AnyBuffer.from_numpy(device, a, dtype) for a in (x, gamma, beta)]
    (y,) = R.run(node, bufs, device)
    return y.to_numpy(shape)


def _ln_bwd(device, dy, x, gamma, eps=1e-5, dtype=F32):
    shape = np.asarray(x).shape
    cols = shape[-1]
    node = Node("LAYER_NORM_GRAD", Layout(*shape), dtype,
                [Node.leaf(Layout(*shape), dtype), Node.leaf(Layout(*shape), dtype), Node.leaf(Layout(cols), dtype)],
                {"eps": eps, "axis": -1})
    bufs = [AnyBuffer.from_numpy(device, a, dtype) for a in (dy, x, gamma)]
    dx, dg, db = R.run(node, bufs, device)
    return dx.to_numpy(shape), dg.to_numpy(), db.to_numpy()


# ---- the reference's golden vectors, through the dispatch surface -------------------


@pytest.mark.parametrize("g", golden("layer_norm_fwd"), ids=lambda g: g["cite"])
def test_fwd_goldens(device, g):
    y = _ln_fwd(device, g["x"], g["gamma"], g["beta"], g["eps"])
    np.testing.assert_allclose(y, g["y"], atol=g["atol"])


@pytest.mark.parametrize("g", golden("layer_norm_bwd"), ids=lambda g: g["cite"])
def test_bwd_goldens(device, g):
    got = dict(zip(("dx", "dgamma", "dbeta"), _ln_bwd(device, g["dy"], g["x"], g["gamma"], g["eps"])))
    checked = [k for k in got if k in g]
    assert checked
    for k in checked:
        np.testing.assert_allclose(got[k], g[k], atol=g["atol"], err_msg=k)


# ---- random shapes: every register layout, the scalar path, the streaming fallback ---

SHAPES = [
    (1, 4), (3, 7), (5, 65), (33, 130), (64, 384), (16, 1000), (9, 1024), (17, 2048), (6, 4096), (5, 8192),
    (3, 16384), (2, 20000), (4, 1023), (2, 40000), (300, 96), (1, 50000),
    # tall and wide: the backward pairs 512-thread rows in 1024-thread workgroups (odd row
    # counts leave a row slot without a row at the end of a group)
    (1027, 4096), (1025, 3000), (1031, 8192),
    # 128 or more row groups: the partial dgamma/dbeta rows are summed by the 32-column slab
    # reduction (133 groups: one full pass of 128 group lanes and a ragged one; 512 groups;
    # 388 and 644 columns leave the last slab ragged)
    (530, 644), (2100, 388), (4300, 388),
]


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_fwd_bwd_random_f32(device, rows, cols):
    cfg = 20
    x = normal(cfg, 0, (rows, cols), std=1.5, mean=0.3)
    g = uniform(cfg, 1, (cols,), 0.5, 1.5)
    b = normal(cfg, 2, (cols,), std=0.1)
    dy = normal(cfg, 3, (rows, cols))
    assert_close(_ln_fwd(device, x, g, b), O.layer_norm_fwd(x, g, b), RTOL_F32, ATOL_F32, "y")
    dx, dg, db = _ln_bwd(device, dy, x, g)
    rdx, rdg, rdb = O.layer_norm_bwd(dy, x, g)
    assert_close(dx, rdx, RTOL_F32, ATOL_F32, "dx")
    mu, rstd = O.layer_norm_stats(x, 1e-5)
    xhat = (x - mu) * rstd
    assert_sum_close(dg, rdg, np.abs(dy * xhat).sum(axis=0), what="dgamma")
    assert_sum_close(db, rdb, np.abs(dy).sum(axis=0), what="dbeta")


def test_large_mean_rows_keep_precision(device):
    # E[x^2] - E[x]^2 in fp32 would lose the variance here
    x = normal(21, 0, (8, 512), std=1.0, mean=300.0)
    g = np.ones(512, np.float32)
    dy = normal(21, 1, (8, 512))
    assert_close(_ln_fwd(device, x, g, np.zeros(512)), O.layer_norm_fwd(x, g, np.zeros(512)), 1e-3, 1e-3, "y")
    dx, _, _ = _ln_bwd(device, dy, x, g)
    assert_close(dx, O.layer_norm_bwd(dy, x, g)[0], 1e-3, 1e-3, "dx")


def test_rank3_input(device):
    x = normal(22, 0, (2, 3, 64))
    dy = normal(22, 1, (2, 3, 64))
    g = uniform(22, 2, (64,), 0.5, 1.5)
    dx, dg, db = _ln_bwd(device, dy, x, g)
    rdx, rdg, rdb = O.layer_norm_bwd(dy, x, g)
    assert_close(dx, rdx, RTOL_F32, ATOL_F32, "dx")
    assert_close(dg, rdg, RTOL_F32, 1e-4, "dgamma")
    assert_close(db, rdb, RTOL_F32, 1e-4, "dbeta")


def test_benchmark_shape_f32(device):
    # LayerNorm (2048, 4096) fp32: x~N(0,1), gamma~U(.5,1.5), beta~N(0,.1), dY~N(0,1)
    rows, cols = 2048, 4096
    x = normal(2, 0, (rows, cols))
    g = uniform(2, 1, (cols,), 0.5, 1.5)
    b = normal(2, 2, (cols,), std=0.1)
    dy = normal(2, 3, (rows, cols))
    assert_close(_ln_fwd(device, x, g, b), O.layer_norm_fwd(x, g, b), RTOL_F32, ATOL_F32, "y")
    dx, dg, db = _ln_bwd(device, dy, x, g)
    rdx, rdg, rdb = O.layer_norm_bwd(dy, x, g)
    assert_close(dx, rdx, RTOL_F32, ATOL_F32, "dx")
    mu, rstd = O.layer_norm_stats(x, 1e-5)
    assert_sum_close(dg, rdg, np.abs(dy * (x - mu) * rstd).sum(axis=0), what="dgamma")
    assert_sum_close(db, rdb, np.abs(dy).sum(axis=0), what="dbeta")
    # size-independent properties: dbeta is the column sum of dy; with gamma = 1 every
    # row of dx sums to zero
    dx1, _, db1 = _ln_bwd(device, dy, x, np.ones(cols, np.float32))
    assert np.max(np.abs(dx1.astype(np.float64).sum(axis=1))) < 1e-3
    np.testing.assert_allclose(db1, db, rtol=0, atol=0)  # same sums, same order: bit-identical


def test_saved_statistics_path(device):
    rows, cols = 257, 1024
    x = normal(23, 0, (rows, cols), mean=-2.0)
    g = uniform(23, 1, (cols,), 0.5, 1.5)
    b = normal(23, 2, (cols,))
    dy = normal(23, 3, (rows, cols))
    bx, bg, bb, bdy = (AnyBuffer.from_numpy(device, a) for a in (x, g, b, dy))
    y = AnyBuffer.create(F32, device, rows * cols)
    mean = AnyBuffer.create(F32, device, rows)
    rstd = AnyBuffer.create(F32, device, rows)
    lib = device.lib
    lib.mg_layer_norm_fwd_stats(bx.data_ptr(), bg.data_ptr(), bb.data_ptr(), y.data_ptr(), mean.data_ptr(),
                                rstd.data_ptr(), rows, cols, 1e-5, F32, device.stream)
    mu, rs = O.layer_norm_stats(x, 1e-5)
    assert_close(mean.to_numpy(), mu[:, 0], RTOL_F32, ATOL_F32, "mean")
    assert_close(rstd.to_numpy(), rs[:, 0], RTOL_F32, ATOL_F32, "rstd")
    dx, dg, db = (AnyBuffer.create(F32, device, n) for n in (rows * cols, cols, cols))
    lib.mg_layer_norm_bwd_stats(bdy.data_ptr(), bx.data_ptr(), bg.data_ptr(), mean.data_ptr(), rstd.data_ptr(),
                                dx.data_ptr(), dg.data_ptr(), db.data_ptr(), rows, cols, F32, device.stream)
    rdx, rdg, rdb = O.layer_norm_bwd(dy, x, g)
    assert_close(dx.to_numpy((rows, cols)), rdx, RTOL_F32, ATOL_F32, "dx")
    assert_sum_close(dg.to_numpy(), rdg, np.abs(dy * (x - mu) * rs).sum(axis=0), what="dgamma")
    assert_sum_close(db.to_numpy(), rdb, np.abs(dy).sum(axis=0), what="dbeta")


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("rows,cols", [(64, 384), (9, 1000), (33, 4096), (5, 16384), (3, 40000), (7, 129), (1027, 4096)])
def test_backward_added_to_a_residual_equals_separate_calls(device, dtype, rows, cols):
    # mg_layer_norm_bwd_stats_add: bit for bit mg_layer_norm_bwd_stats followed by mg_add, with
    # the residual in its own buffer and with the residual being dx itself (accumulation in
    # place); every row layout incl. the streaming fallback for very wide rows.
    lib, st = device.lib, device.stream
    P = lambda b: b.data_ptr()
    x = round_to_dtype(normal(24, 0, (rows, cols)), dtype)
    g = round_to_dtype(uniform(24, 1, (cols,), 0.5, 1.5), dtype)
    b = round_to_dtype(normal(24, 2, (cols,)), dtype)
    dy = round_to_dtype(normal(24, 3, (rows, cols)), dtype)
    res = round_to_dtype(normal(24, 4, (rows, cols)), dtype)
    bx, bg, bb, bdy, bres = (AnyBuffer.from_numpy(device, a, dtype) for a in (x, g, b, dy, res))
    n = rows * cols
    y, mean, rstd = AnyBuffer.create(dtype, device, n), AnyBuffer.create(F32, device, rows), AnyBuffer.create(F32, device, rows)
    lib.mg_layer_norm_fwd_stats(P(bx), P(bg), P(bb), P(y), P(mean), P(rstd), rows, cols, 1e-5, dtype, st)
    dx, dg, db, want = (AnyBuffer.create(dtype, device, m) for m in (n, cols, cols, n))
    lib.mg_layer_norm_bwd_stats(P(bdy), P(bx), P(bg), P(mean), P(rstd), P(dx), P(dg), P(db), rows, cols, dtype, st)
    lib.mg_add(P(dx), P(bres), P(want), n, dtype, st)
    got, dg2, db2 = (AnyBuffer.create(dtype, device, m) for m in (n, cols, cols))
    lib.mg_layer_norm_bwd_stats_add(P(bdy), P(bx), P(bg), P(mean), P(rstd), P(bres), P(got), P(dg2), P(db2), rows, cols,
                                    dtype, st)
    np.testing.assert_array_equal(got.to_numpy(), want.to_numpy())
    np.testing.assert_array_equal(dg2.to_numpy(), dg.to_numpy())
    np.testing.assert_array_equal(db2.to_numpy(), db.to_numpy())
    inplace = AnyBuffer.from_numpy(device, res, dtype)
    lib.mg_layer_norm_bwd_stats_add(P(bdy), P(bx), P(bg), P(mean), P(rstd), P(inplace), P(inplace), P(dg2), P(db2), rows,
                                    cols, dtype, st)
    np.testing.assert_array_equal(inplace.to_numpy(), want.to_numpy())


@pytest.mark.parametrize("dtype,rtol,atol", [(F16, 2e-3, 2e-3), (BF16, 1.6e-2, 1.6e-2)])
@pytest.mark.parametrize("rows,cols", [(64, 384), (8, 1000), (33, 4096), (5, 16384), (3, 40000)])
def test_half_precision_storage(device, dtype, rtol, atol, rows, cols):
    # Inputs are rounded once to the storage type; the oracle sees the rounded values.
    # The bound is the storage type's rounding of the result (2^-11 / 2^-8 relative).
    x = round_to_dtype(normal(24, 0, (rows, cols)), dtype)
    g = round_to_dtype(uniform(24, 1, (cols,), 0.5, 1.5), dtype)
    b = round_to_dtype(normal(24, 2, (cols,), std=0.1), dtype)
    dy = round_to_dtype(normal(24, 3, (rows, cols)), dtype)
    assert_close(_ln_fwd(device, x, g, b, dtype=dtype), O.layer_norm_fwd(x, g, b), rtol, atol, "y")
    dx, dg, db = _ln_bwd(device, dy, x, g, dtype=dtype)
    rdx, rdg, rdb = O.layer_norm_bwd(dy, x, g)
    assert_close(dx, rdx, rtol, atol, "dx")
    assert_close(dg, rdg, rtol, atol * 4, "dgamma")
    assert_close(db, rdb, rtol, atol * 4, "dbeta")


def test_outputs_do_not_depend_on_prior_contents(device):
    # dgamma/dbeta are overwritten, not accumulated into (the reference zero-fills them
    # in the caller; this library must not rely on that)
    rows, cols = 40, 256
    x, dy = normal(25, 0, (rows, cols)), normal(25, 1, (rows, cols))
    g = uniform(25, 2, (cols,), 0.5, 1.5)
    bx, bdy, bg = (AnyBuffer.from_numpy(device, a) for a in (x, dy, g))
    outs = []
    for fill in (0.0, 1e30):
        dx = AnyBuffer.create(F32, device, rows * cols, fill=fill)
        dg = AnyBuffer.create(F32, device, cols, fill=fill)
        db = AnyBuffer.create(F32, device, cols, fill=fill)
        device.lib.mg_layer_norm_bwd(bdy.data_ptr(), bx.data_ptr(), bg.data_ptr(), dx.data_ptr(), dg.data_ptr(),
                                     db.data_ptr(), rows, cols, 1e-5, F32, device.stream)
        outs.append((dx.to_numpy(), dg.to_numpy(), db.to_numpy()))
    for a, b in zip(*outs):
        np.testing.assert_array_equal(a, b)


def test_errors(device):
    buf = AnyBuffer.create(F32, device, 16)
    p = buf.data_ptr()
    with pytest.raises(MogradError, match="unsupported dtype"):
        device.lib.mg_layer_norm_fwd(p, p, p, p, 4, 4, 1e-5, R.int64, device.stream)
    with pytest.raises(MogradError, match="bad shape"):
        device.lib.mg_layer_norm_bwd(p, p, p, p, p, p, 4, 0, 1e-5, F32, device.stream)
    with pytest.raises(MogradError, match="null"):
        device.lib.mg_layer_norm_bwd(p, None, p, p, p, p, 4, 4, 1e-5, F32, device.stream)
