"""Matmul family and Linear gradients on the GPU against the float64 oracle.

The operand layouts are the ones mograd's graph produces for a Linear layer
(mograd/grad.mojo:180-187, mograd/runtime/gpu/rewrites.mojo:163-174): forward
X W^T + b, dX = MATMUL_BT(dY, TRANSPOSE(W)) with a strided right operand, and
dW^T = MATMUL(TRANSPOSE(X), dY) with a strided left operand; db = SUM(axis=0).
"""
import ctypes as C

import numpy as np
import pytest

from helpers import ATOL_F32, RTOL_F32, assert_close, assert_sum_close, normal, uniform
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu

from mograd_amd import BF16, F16, F32, AnyBuffer, Layout, MogradError, Node  # noqa: E402
from mograd_amd import runtime as R  # noqa: E402
from mograd_amd.runtime import round_to_dtype  # noqa: E402


def _run(device, op, out_layout, operands, dtype=F32, attrs=None):
    """operands: list of (host array, layout view over it)."""
    srcs = [Node.leaf(l, dtype) for _, l in operands]
    node = Node(op, out_layout, dtype, srcs, attrs or {})
    bufs = [AnyBuffer.from_numpy(device, a, dtype).view(l) for a, l in operands]
    (out,) = R.run(node, bufs, device)
    return out.to_numpy(out_layout.shape())


def _linear_all(device, x, w, b, dy, dtype=F32):
    """Forward and the three gradients, each through the scheduler entry the reference's
    graph reaches."""
    M, K = x.shape
    N = w.shape[0]
    y = _run(device, "MATMUL_BIAS_BT", Layout(M, N), [(x, Layout(M, K)), (w, Layout(N, K)), (b, Layout(N))], dtype)
    # dX = MATMUL_BT(dY, W^T view): the right operand is the (K, N) transposed view of W
    dx = _run(device, "MATMUL_BT", Layout(M, K), [(dy, Layout(M, N)), (w, Layout(N, K).transpose())], dtype)
    # dW^T = MATMUL(X^T view, dY), shape (K, N)
    dwt = _run(device, "MATMUL", Layout(K, N), [(x, Layout(M, K).transpose()), (dy, Layout(M, N))], dtype)
    db = _run(device, "SUM", Layout(N), [(dy, Layout(M, N))], dtype, {"axis": 0})
    return y, dx, dwt.T, db


SHAPES = [(64, 10, 256), (64, 256, 784), (128, 128, 128), (256, 384, 512), (200, 136, 260), (130, 65, 384),
          (1, 8, 16), (33, 7, 5), (512, 1024, 256), (300, 128, 1000),
          # a 10-class head behind a wide layer: few output tiles (split along K in fp32) and a
          # 10-wide gradient that is copied k-contiguous before the tiled kernel reads it
          (2048, 10, 4096), (1024, 6, 1024), (640, 12, 2080)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_linear_fwd_and_grads_f32(device, M, N, K):
    x = normal(40, 0, (M, K))
    bound = np.sqrt(6.0 / K)
    w = uniform(40, 1, (N, K), -bound, bound)
    b = uniform(40, 2, (N,), -bound, bound)
    dy = normal(40, 3, (M, N))
    y, dx, dw, db = _linear_all(device, x, w, b, dy)
    # each output is a dot product of length K, N or M: tolerance at the parity rtol
    # against the value, with the absolute floor scaled by the dot product's L1 mass
    assert_sum_close(y, O.matmul_bias_bt(x, w, b), np.abs(x) @ np.abs(w).T, what="y")
    assert_sum_close(dx, O.linear_grad_x(dy, w), np.abs(dy) @ np.abs(w), what="dx")
    assert_sum_close(dw, O.linear_grad_w(dy, x), np.abs(dy).T @ np.abs(x), what="dw")
    assert_sum_close(db, O.linear_grad_b(dy), np.abs(dy).sum(axis=0), what="db")


@pytest.mark.parametrize("M,N,K", [(128, 256, 512), (200, 136, 260), (64, 10, 256), (2048, 10, 4096), (1024, 6, 512)])
def test_linear_bwd_entry(device, M, N, K):
    x, w, dy = normal(41, 0, (M, K)), normal(41, 1, (N, K)), normal(41, 2, (M, N))
    bx, bw, bdy = (AnyBuffer.from_numpy(device, a) for a in (x, w, dy))
    dx, dw, db = (AnyBuffer.create(F32, device, n) for n in (M * K, N * K, N))
    device.lib.mg_linear_bwd(bdy.data_ptr(), bx.data_ptr(), bw.data_ptr(), dx.data_ptr(), dw.data_ptr(),
                             db.data_ptr(), M, N, K, F32, device.stream)
    assert_sum_close(dx.to_numpy((M, K)), O.linear_grad_x(dy, w), np.abs(dy) @ np.abs(w), what="dx")
    assert_sum_close(dw.to_numpy((N, K)), O.linear_grad_w(dy, x), np.abs(dy).T @ np.abs(x), what="dw")
    assert_sum_close(db.to_numpy(), O.linear_grad_b(dy), np.abs(dy).sum(axis=0), what="db")


def test_batched_rank3_and_broadcast_weight(device):
    # (B, T, K) activations against one (N, K) weight: the GPT's Linear layers
    Bt, T, K, N = 3, 40, 64, 96
    x = normal(42, 0, (Bt, T, K))
    w = normal(42, 1, (N, K))
    out = _run(device, "MATMUL_BT", Layout(Bt, T, N),
               [(x, Layout(Bt, T, K)), (w, Layout(Bt, N, K, strides=(0, K, 1)))])
    assert_sum_close(out, np.einsum("btk,nk->btn", x.astype(np.float64), w), 
                     np.einsum("btk,nk->btn", np.abs(x), np.abs(w)), what="batched")


def test_batched_thin_products_f32(device):
    # three (T, K) x (K, 10) products and their transposed-operand gradients in one call each:
    # the split along K and the k-contiguous copy both carry the batch index
    Bt, T, K, N = 3, 256, 2048, 10
    x, w, dy = normal(43, 0, (Bt, T, K)), normal(43, 1, (Bt, N, K)), normal(43, 2, (Bt, T, N))
    y = _run(device, "MATMUL_BT", Layout(Bt, T, N), [(x, Layout(Bt, T, K)), (w, Layout(Bt, N, K))])
    assert_sum_close(y, np.einsum("btk,bnk->btn", x.astype(np.float64), w),
                     np.einsum("btk,bnk->btn", np.abs(x), np.abs(w)), what="y")
    # dW^T = X^T dY per batch: the (T, 10) right operand is read along T
    dwt = _run(device, "MATMUL", Layout(Bt, K, N),
               [(x, Layout(Bt, K, T, strides=(T * K, 1, K))), (dy, Layout(Bt, T, N))])
    assert_sum_close(dwt, np.einsum("btk,btn->bkn", x.astype(np.float64), dy),
                     np.einsum("btk,btn->bkn", np.abs(x), np.abs(dy)), what="dwt")
    # dW = dY^T X per batch: the (10, T) left operand is the transposed view of dY
    dw = _run(device, "MATMUL", Layout(Bt, N, K),
              [(dy, Layout(Bt, N, T, strides=(T * N, 1, N))), (x, Layout(Bt, T, K))])
    assert_sum_close(dw, np.einsum("btn,btk->bnk", dy.astype(np.float64), x),
                     np.einsum("btn,btk->bnk", np.abs(dy), np.abs(x)), what="dw")


def test_mlp_chain_matches_oracle(device):
    # MNIST-shaped MLP 64x784 -> 256 (ReLU) -> 10, CE on labels: the whole gradient chain
    # CE grad -> dW2, db2, dX -> ReLU grad -> dW1, db1
    M, D0, D1, D2 = 64, 784, 256, 10
    x = normal(1, 0, (M, D0))
    w1 = uniform(1, 1, (D1, D0), -np.sqrt(6 / D0), np.sqrt(6 / D0))
    b1 = uniform(1, 2, (D1,), -np.sqrt(6 / D0), np.sqrt(6 / D0))
    w2 = uniform(1, 3, (D2, D1), -np.sqrt(6 / D1), np.sqrt(6 / D1))
    b2 = uniform(1, 4, (D2,), -np.sqrt(6 / D1), np.sqrt(6 / D1))
    ids = np.random.Generator(np.random.PCG64(1005)).integers(0, D2, M)
    onehot = O.one_hot(ids, D2).astype(np.float32)
    # oracle
    h_pre = O.matmul_bias_bt(x, w1, b1)
    h = np.maximum(h_pre, 0)
    logits = O.matmul_bias_bt(h, w2, b2)
    want_loss = O.cross_entropy(logits, onehot)
    dlogits = O.cross_entropy_grad(logits, onehot)
    want = {"dw2": O.linear_grad_w(dlogits, h), "db2": O.linear_grad_b(dlogits)}
    dh = O.relu_grad(h, O.linear_grad_x(dlogits, w2))
    want.update({"dw1": O.linear_grad_w(dh, x), "db1": O.linear_grad_b(dh)})
    # GPU, buffers stay on the device between ops
    lib, st = device.lib, device.stream
    up = lambda a: AnyBuffer.from_numpy(device, a)  # noqa: E731
    bx, bw1, bb1, bw2, bb2, by = up(x), up(w1), up(b1), up(w2), up(b2), up(onehot)
    one = up(np.ones(1, np.float32))
    new = lambda n: AnyBuffer.create(F32, device, n)  # noqa: E731
    hpre, hb, lg, loss, dlg = new(M * D1), new(M * D1), new(M * D2), new(1), new(M * D2)
    lib.mg_matmul_bias_bt(bx.data_ptr(), bw1.data_ptr(), bb1.data_ptr(), hpre.data_ptr(), 1, M, D1, D0, D0, 1, D0, 1,
                          M * D0, D1 * D0, F32, st)
    # relu forward is outside this path: relu(h_pre) == relu_grad(h_pre, h_pre)
    lib.mg_relu_grad(hpre.data_ptr(), hpre.data_ptr(), hb.data_ptr(), M * D1, F32, st)
    lib.mg_matmul_bias_bt(hb.data_ptr(), bw2.data_ptr(), bb2.data_ptr(), lg.data_ptr(), 1, M, D2, D1, D1, 1, D1, 1,
                          M * D1, D2 * D1, F32, st)
    lib.mg_cross_entropy(lg.data_ptr(), by.data_ptr(), loss.data_ptr(), M, D2, F32, st)
    lib.mg_cross_entropy_grad(lg.data_ptr(), by.data_ptr(), one.data_ptr(), dlg.data_ptr(), M, D2, F32, st)
    dw2, db2, dhb, dh2, dw1, db1 = new(D2 * D1), new(D2), new(M * D1), new(M * D1), new(D1 * D0), new(D1)
    lib.mg_linear_bwd(dlg.data_ptr(), hb.data_ptr(), bw2.data_ptr(), dhb.data_ptr(), dw2.data_ptr(), db2.data_ptr(),
                      M, D2, D1, F32, st)
    lib.mg_relu_grad(hb.data_ptr(), dhb.data_ptr(), dh2.data_ptr(), M * D1, F32, st)
    lib.mg_linear_bwd(dh2.data_ptr(), bx.data_ptr(), bw1.data_ptr(), None, dw1.data_ptr(), db1.data_ptr(), M, D1, D0,
                      F32, st)
    assert_close(loss.item(), want_loss, RTOL_F32, ATOL_F32, "loss")
    got = {"dw2": dw2.to_numpy((D2, D1)), "db2": db2.to_numpy(), "dw1": dw1.to_numpy((D1, D0)), "db1": db1.to_numpy()}
    for k in want:
        assert_close(got[k], want[k], RTOL_F32, ATOL_F32, k)


def test_readme_mlp_square_layer_f32(device):
    # The 4096 -> 4096 Linear of the README MLP at batch 2048: forward, dX, dW, db at the
    # size where 1024 output tiles are walked by a grid of 512 resident workgroups.
    M = 2048
    N = K = 4096
    x = normal(3, 30, (M, K))
    bound = np.sqrt(6.0 / K)
    w = uniform(3, 31, (N, K), -bound, bound)
    b = uniform(3, 32, (N,), -bound, bound)
    dy = normal(3, 33, (M, N))
    y, dx, dw, db = _linear_all(device, x, w, b, dy)
    assert_sum_close(y, O.matmul_bias_bt(x, w, b), np.abs(x) @ np.abs(w).T, what="y")
    assert_sum_close(dx, O.linear_grad_x(dy, w), np.abs(dy) @ np.abs(w), what="dx")
    assert_sum_close(dw, O.linear_grad_w(dy, x), np.abs(dy).T @ np.abs(x), what="dw")
    assert_sum_close(db, O.linear_grad_b(dy), np.abs(dy).sum(axis=0), what="db")


def test_readme_mlp_chain_matches_oracle(device):
    # README MLP, fp32: x (2048,4096) -> Linear 4096 +ReLU -> LayerNorm -> Linear 4096 +ReLU ->
    # Linear 10 -> cross-entropy on integer labels; the call sequence of the benchmark's
    # MLP step, every gradient against the float64 oracle chain.
    from mograd_amd import I32

    lib, st = device.lib, device.stream
    M, D, NC = 2048, 4096, 10
    bound = np.sqrt(6.0 / D)
    x = normal(3, 0, (M, D))
    w1, w2 = (uniform(3, i, (D, D), -bound, bound) for i in (1, 3))
    b1, b2 = (uniform(3, i, (D,), -bound, bound) for i in (2, 4))
    w3, b3 = uniform(3, 5, (NC, D), -bound, bound), uniform(3, 6, (NC,), -bound, bound)
    gamma, beta = np.ones(D, np.float32), np.zeros(D, np.float32)
    ids = np.random.Generator(np.random.PCG64(3007)).integers(0, NC, M).astype(np.int32)
    up = lambda a: AnyBuffer.from_numpy(device, a)  # noqa: E731
    new = lambda n: AnyBuffer.create(F32, device, n)  # noqa: E731
    P = lambda t: t.data_ptr()  # noqa: E731
    bx, bw1, bw2, bw3, bb1, bb2, bb3, bg, bbt = (up(a) for a in (x, w1, w2, w3, b1, b2, b3, gamma, beta))
    bids = AnyBuffer.from_numpy(device, ids, I32)
    h1p, h1, ln, h2p, h2, logits = new(M * D), new(M * D), new(M * D), new(M * D), new(M * D), new(M * NC)
    loss, dlogits = new(1), new(M * NC)
    dh2, dh2p, dln, dh1, dh1p = new(M * D), new(M * D), new(M * D), new(M * D), new(M * D)
    dw1, dw2, dw3, db1, db2, db3, dg, dbt = new(D * D), new(D * D), new(NC * D), new(D), new(D), new(NC), new(D), new(D)

    def linear(a, w, b, y, n_out, k):
        lib.mg_matmul_bias_bt(P(a), P(w), P(b), P(y), 1, M, n_out, k, k, 1, k, 1, M * k, n_out * k, F32, st)

    linear(bx, bw1, bb1, h1p, D, D)
    lib.mg_relu_grad(P(h1p), P(h1p), P(h1), M * D, F32, st)  # relu(v) == relu_grad(v, v)
    lib.mg_layer_norm_fwd(P(h1), P(bg), P(bbt), P(ln), M, D, 1e-5, F32, st)
    linear(ln, bw2, bb2, h2p, D, D)
    lib.mg_relu_grad(P(h2p), P(h2p), P(h2), M * D, F32, st)
    linear(h2, bw3, bb3, logits, NC, D)
    lib.mg_cross_entropy_fused_ids(P(logits), P(bids), None, P(loss), P(dlogits), M, NC, F32, I32, st)
    lib.mg_linear_bwd(P(dlogits), P(h2), P(bw3), P(dh2), P(dw3), P(db3), M, NC, D, F32, st)
    lib.mg_relu_grad(P(h2), P(dh2), P(dh2p), M * D, F32, st)
    lib.mg_linear_bwd(P(dh2p), P(ln), P(bw2), P(dln), P(dw2), P(db2), M, D, D, F32, st)
    lib.mg_layer_norm_bwd(P(dln), P(h1), P(bg), P(dh1), P(dg), P(dbt), M, D, 1e-5, F32, st)
    lib.mg_relu_grad(P(h1), P(dh1), P(dh1p), M * D, F32, st)
    lib.mg_linear_bwd(P(dh1p), P(bx), P(bw1), None, P(dw1), P(db1), M, D, D, F32, st)

    # Oracle chain in float64.  A pre-activation within rounding of zero has no determined
    # sign: there (and only there) the oracle takes the mask the fp32 forward produced.
    def mask_of(pre64, pre_gpu, what):
        m64 = pre64 > 0
        unsure = np.abs(pre64) < 1e-4
        assert np.array_equal(m64[~unsure], (pre_gpu > 0)[~unsure]), what
        assert unsure.mean() < 1e-3, what
        return np.where(unsure, pre_gpu > 0, m64)

    r_h1p = O.matmul_bias_bt(x, w1, b1)
    g_h1p = h1p.to_numpy((M, D))
    assert_sum_close(g_h1p, r_h1p, np.abs(x) @ np.abs(w1).T, what="h1 pre-activation")
    m1 = mask_of(r_h1p, g_h1p, "relu 1 mask")
    r_h1 = np.where(m1, r_h1p, 0.0)
    r_ln = O.layer_norm_fwd(r_h1, gamma, beta)
    # the LayerNorm's input carries the rounding of the product before it, scaled by rstd
    _, rstd1 = O.layer_norm_stats(r_h1, 1e-5)
    assert_sum_close(ln.to_numpy((M, D)), r_ln, rstd1 * (np.abs(x) @ np.abs(w1).T), what="layer norm output")
    r_h2p = O.matmul_bias_bt(r_ln, w2, b2)
    g_h2p = h2p.to_numpy((M, D))
    m2 = mask_of(r_h2p, g_h2p, "relu 2 mask")
    r_h2 = np.where(m2, r_h2p, 0.0)
    r_logits = O.matmul_bias_bt(r_h2, w3, b3)
    assert_sum_close(logits.to_numpy((M, NC)), r_logits, np.abs(r_h2) @ np.abs(w3).T, what="logits")
    assert_close(loss.item(), O.cross_entropy_ids(r_logits, ids), RTOL_F32, ATOL_F32, "loss")
    r_dlogits = O.cross_entropy_grad_ids(r_logits, ids)
    a = np.abs
    assert_sum_close(dw3.to_numpy((NC, D)), O.linear_grad_w(r_dlogits, r_h2), a(r_dlogits).T @ a(r_h2), what="dw3")
    assert_sum_close(db3.to_numpy(), O.linear_grad_b(r_dlogits), a(r_dlogits).sum(axis=0), what="db3")
    r_dh2p = np.where(m2, O.linear_grad_x(r_dlogits, w3), 0.0)
    assert_sum_close(dw2.to_numpy((D, D)), O.linear_grad_w(r_dh2p, r_ln), a(r_dh2p).T @ a(r_ln), what="dw2")
    assert_sum_close(db2.to_numpy(), O.linear_grad_b(r_dh2p), a(r_dh2p).sum(axis=0), what="db2")
    r_dln = O.linear_grad_x(r_dh2p, w2)
    assert_sum_close(dln.to_numpy((M, D)), r_dln, a(r_dh2p) @ a(w2), what="dln")
    r_dh1, r_dg, r_dbt = O.layer_norm_bwd(r_dln, r_h1, gamma)
    xhat = O.layer_norm_fwd(r_h1, gamma, beta)
    assert_sum_close(dg.to_numpy(), r_dg, (a(r_dln) * a(xhat)).sum(axis=0), what="dgamma")
    assert_sum_close(dbt.to_numpy(), r_dbt, a(r_dln).sum(axis=0), what="dbeta")
    # dx of a LayerNorm row: rstd * (dy - mean(dy) - xhat * mean(dy * xhat)), each mean a sum of
    # 4096 terms of the size of dln
    row = a(r_dln).mean(axis=1, keepdims=True)
    assert_sum_close(dh1.to_numpy((M, D)), r_dh1, rstd1 * (a(r_dln) + row * (1.0 + a(xhat))), what="dh1")
    r_dh1p = np.where(m1, r_dh1, 0.0)
    assert_sum_close(dw1.to_numpy((D, D)), O.linear_grad_w(r_dh1p, x), a(r_dh1p).T @ a(x), what="dw1")
    assert_sum_close(db1.to_numpy(), O.linear_grad_b(r_dh1p), a(r_dh1p).sum(axis=0), what="db1")


@pytest.mark.parametrize("dtype,rtol", [(F16, 2e-3), (BF16, 1.6e-2)])
def test_half_precision_storage(device, dtype, rtol):
    M, N, K = 96, 80, 136
    x = round_to_dtype(normal(43, 0, (M, K)), dtype)
    w = round_to_dtype(normal(43, 1, (N, K), std=0.1), dtype)
    b = round_to_dtype(normal(43, 2, (N,), std=0.1), dtype)
    dy = round_to_dtype(normal(43, 3, (M, N)), dtype)
    y, dx, dw, db = _linear_all(device, x, w, b, dy, dtype)
    for got, want, name in ((y, O.matmul_bias_bt(x, w, b), "y"), (dx, O.linear_grad_x(dy, w), "dx"),
                            (dw, O.linear_grad_w(dy, x), "dw"), (db, O.linear_grad_b(dy), "db")):
        assert_close(got, want, rtol, rtol * np.abs(want).max(), name)


def test_sum_axis_shapes(device):
    for shape, axis in [((2048, 4096), 0), ((7, 5), 0), ((3, 50, 8), 1), ((4, 6, 10), 2), ((1000, 3), 0), ((2, 3, 4), 0)]:
        a = normal(44, len(shape) * 10 + axis, shape)
        out_shape = tuple(s for i, s in enumerate(shape) if i != axis)
        got = _run(device, "SUM", Layout(*out_shape), [(a, Layout(*shape))], F32, {"axis": axis})
        assert_sum_close(got, a.astype(np.float64).sum(axis=axis), np.abs(a).sum(axis=axis), what=f"sum{shape}/{axis}")


def test_sum_axis_wide_one_launch(device):
    # Wide matrices (at least 128 column slabs of 128 bytes) are summed by one launch, a
    # workgroup per slab: ragged row counts, a ragged last slab, a batch of two, an exact
    # integer sum, and the same column sums whatever the slab kernel's row order.
    for shape, axis in [((1000, 4100), 0), ((129, 8200), 0), ((2, 300, 4096), 1), ((2048, 4096), 0)]:
        a = normal(48, len(shape) * 10 + axis + shape[-1] % 7, shape)
        out_shape = tuple(s for i, s in enumerate(shape) if i != axis)
        got = _run(device, "SUM", Layout(*out_shape), [(a, Layout(*shape))], F32, {"axis": axis})
        assert_sum_close(got, a.astype(np.float64).sum(axis=axis), np.abs(a).sum(axis=axis), what=f"sum{shape}/{axis}")
    # small integers: every partial sum is exact in fp32, so the result is the integer sum
    rows, cols = 1153, 4128
    a = (np.arange(rows * cols, dtype=np.int64).reshape(rows, cols) * 7919 % 17 - 8).astype(np.float32)
    got = _run(device, "SUM", Layout(cols), [(a, Layout(rows, cols))], F32, {"axis": 0})
    np.testing.assert_array_equal(got, a.astype(np.int64).sum(axis=0).astype(np.float32))
    for dtype, rtol in ((F16, 2e-3), (BF16, 1.6e-2)):
        a = round_to_dtype(normal(48, 5, (1031, 8200)), dtype)
        got = _run(device, "SUM", Layout(8200), [(a, Layout(1031, 8200))], dtype, {"axis": 0})
        want = a.astype(np.float64).sum(axis=0)
        assert_close(got, want, rtol, rtol * np.abs(want).max(), f"sum 16-bit {dtype}")


def test_relu_grad(device):
    for n in (1, 7, 4096, 100003):
        out = np.maximum(normal(45, n % 97, (n,)), 0)
        up = normal(45, 1 + n % 97, (n,))
        got = _run(device, "RELU_GRAD", Layout(n), [(out, Layout(n)), (up, Layout(n))])
        np.testing.assert_array_equal(got, O.relu_grad(out, up).astype(np.float32))  # a select: bit-exact


def test_errors(device):
    a = normal(46, 0, (2, 3, 4, 5))
    with pytest.raises(MogradError, match="non-collapsible batch dims"):
        # transpose(1, 2) of a rank-4 tensor: batch dims no longer fold into one stride
        _run(device, "MATMUL", Layout(2, 4, 3, 3),
             [(a, Layout(2, 3, 4, 5).transpose(1, 2)), (a, Layout(2, 3, 4, 5).transpose(1, 2).transpose(2, 3))])
    buf = AnyBuffer.create(F32, device, 16)
    p = buf.data_ptr()
    with pytest.raises(MogradError, match="unsupported dtype"):
        device.lib.mg_matmul(p, p, p, 1, 2, 2, 2, 2, 1, 2, 1, 4, 4, R.int64, device.stream)
    with pytest.raises(MogradError, match="null bias"):
        device.lib.mg_matmul_bias_bt(p, p, None, p, 1, 2, 2, 2, 2, 1, 2, 1, 4, 4, F32, device.stream)


# ---- 16-bit storage on the matrix cores (shapes that take the MFMA kernels) ------------

HALF_MFMA_SHAPES = [(256, 384, 512), (384, 128, 1536), (200, 136, 264), (128, 64, 4096), (4096, 128, 128),
                    (1024, 384, 384), (72, 1536, 384),
                    # extents that are not multiples of 8 (a 65-symbol vocabulary): element-wise staging
                    (2048, 65, 384), (333, 65, 129), (130, 77, 1031), (4099, 65, 384)]


@pytest.mark.parametrize("dtype,rtol", [(F16, 2e-3), (BF16, 1.6e-2)])
@pytest.mark.parametrize("M,N,K", HALF_MFMA_SHAPES)
def test_half_precision_mfma_paths(device, dtype, rtol, M, N, K):
    # forward (k,k), dX (k,n), dW (m,n) operand layouts; dW of the tall shapes is split
    # along K.  Error bound: the storage type's rounding of the result, relative to the
    # largest entry (inputs are rounded once; the oracle sees the rounded values).
    x = round_to_dtype(normal(47, 0, (M, K)), dtype)
    w = round_to_dtype(normal(47, 1, (N, K), std=0.05), dtype)
    b = round_to_dtype(normal(47, 2, (N,), std=0.1), dtype)
    dy = round_to_dtype(normal(47, 3, (M, N), std=0.5), dtype)
    y, dx, dw, db = _linear_all(device, x, w, b, dy, dtype)
    for got, want, name in ((y, O.matmul_bias_bt(x, w, b), "y"), (dx, O.linear_grad_x(dy, w), "dx"),
                            (dw, O.linear_grad_w(dy, x), "dw"), (db, O.linear_grad_b(dy), "db")):
        assert_close(got, want, rtol, rtol * np.abs(want).max(), name)


@pytest.mark.parametrize("dtype,rtol", [(F16, 2e-3), (BF16, 1.6e-2)])
@pytest.mark.parametrize("M,N,K", [(256, 384, 512), (384, 128, 1536), (200, 136, 256), (128, 64, 4096), (1024, 384, 1024),
                                   (72, 1536, 64), (520, 264, 320)])
def test_tile_staging_variants_agree(device, monkeypatch, dtype, rtol, M, N, K):
    # The 16-bit products have a register-staged kernel (0) and one whose tiles are copied
    # straight into LDS, 32 or 64 k per step (322, 642), also with 256 x 128 output tiles
    # (2322, 2642) or 256 x 256 tiles of 128 x 128 wave tiles (4324, 4642); the library picks by operand layout, K and size.  All accumulate each output element over k in the same order on the same MFMA,
    # so forcing either must not change a bit, for every operand layout (forward k/k, dX
    # k/n, dW m/n, the last split along K for the tall shapes) and at ragged tile edges.
    x = round_to_dtype(normal(49, 0, (M, K)), dtype)
    w = round_to_dtype(normal(49, 1, (N, K), std=0.05), dtype)
    b = round_to_dtype(normal(49, 2, (N,), std=0.1), dtype)
    dy = round_to_dtype(normal(49, 3, (M, N), std=0.5), dtype)
    results = {}
    for variant in ("0", "322", "642", "2322", "2642", "4324", "4642"):
        monkeypatch.setenv("MOGRAD_HIP_GEMM16_PIPE", variant)
        results[variant] = _linear_all(device, x, w, b, dy, dtype)
    monkeypatch.delenv("MOGRAD_HIP_GEMM16_PIPE")
    results["auto"] = _linear_all(device, x, w, b, dy, dtype)
    for variant in ("322", "642", "2322", "2642", "4324", "4642", "auto"):
        for got, base, name in zip(results[variant], results["0"], ("y", "dx", "dw", "db")):
            np.testing.assert_array_equal(got, base, err_msg=f"{name}, variant {variant}")
    y, dx, dw, _ = results["auto"]
    for got, want, name in ((y, O.matmul_bias_bt(x, w, b), "y"), (dx, O.linear_grad_x(dy, w), "dx"),
                            (dw, O.linear_grad_w(dy, x), "dw")):
        assert_close(got, want, rtol, rtol * np.abs(want).max(), name)


def test_bf16_linear_bwd_entry_gpt_shapes(device):
    # (tokens, d_model) x (d_ff, d_model): the GPT block's MLP up-projection, scaled down
    M, N, K = 2048, 1536, 384
    x = round_to_dtype(normal(48, 0, (M, K)), BF16)
    w = round_to_dtype(normal(48, 1, (N, K), std=0.05), BF16)
    dy = round_to_dtype(normal(48, 2, (M, N), std=0.5), BF16)
    bx, bw, bdy = (AnyBuffer.from_numpy(device, a, BF16) for a in (x, w, dy))
    dx, dw, db = (AnyBuffer.create(BF16, device, n) for n in (M * K, N * K, N))
    device.lib.mg_linear_bwd(bdy.data_ptr(), bx.data_ptr(), bw.data_ptr(), dx.data_ptr(), dw.data_ptr(),
                             db.data_ptr(), M, N, K, BF16, device.stream)
    for got, want, name in ((dx.to_numpy((M, K)), O.linear_grad_x(dy, w), "dx"),
                            (dw.to_numpy((N, K)), O.linear_grad_w(dy, x), "dw"),
                            (db.to_numpy(), O.linear_grad_b(dy), "db")):
        assert_close(got, want, 1.6e-2, 1.6e-2 * np.abs(want).max(), name)


@pytest.mark.parametrize("dtype,rtol", [(F16, 2e-3), (BF16, 1.6e-2)])
@pytest.mark.parametrize("M,d", [(2048, 96), (1500, 72), (300, 65)])
def test_batched_projections_share_an_operand(device, dtype, rtol, M, d):
    # Three projections of one activation (the Q, K and V of an attention block) as one
    # batched call with batch stride 0 on the shared operand, and their three weight
    # gradients dW_b = dY_b^T X as one batched product that is split along K (= tokens).
    lib, st = device.lib, device.stream
    x = round_to_dtype(normal(53, 0, (M, d)), dtype)
    w = round_to_dtype(normal(53, 1, (3, d, d), std=0.1), dtype)
    dy = round_to_dtype(normal(53, 2, (3, M, d), std=0.5), dtype)
    bx, bw, bdy = (AnyBuffer.from_numpy(device, a, dtype) for a in (x, w, dy))
    y, dw = AnyBuffer.create(dtype, device, 3 * M * d), AnyBuffer.create(dtype, device, 3 * d * d)
    lib.mg_matmul_bt(bx.data_ptr(), bw.data_ptr(), y.data_ptr(), 3, M, d, d, d, 1, d, 1, 0, d * d, dtype, st)
    # A = dY_b^T: element (o, t) at dy_b[t * d + o]; B = X: element (t, i) at x[t * d + i]
    lib.mg_matmul(bdy.data_ptr(), bx.data_ptr(), dw.data_ptr(), 3, d, d, M, 1, d, d, 1, M * d, 0, dtype, st)
    want_y = np.einsum("tk,bnk->btn", x.astype(np.float64), w.astype(np.float64))
    want_dw = np.einsum("bto,ti->boi", dy.astype(np.float64), x.astype(np.float64))
    assert_close(y.to_numpy((3, M, d)), want_y, rtol, rtol * np.abs(want_y).max(), "y")
    assert_close(dw.to_numpy((3, d, d)), want_dw, rtol, rtol * np.abs(want_dw).max(), "dw")


@pytest.mark.parametrize("M,N,K", [(256, 384, 512), (200, 136, 256), (128, 64, 4096), (520, 264, 320), (64, 1000, 32),
                                   (2048, 512, 1024),
                                   # 1024 output tiles: more than the resident workgroups, each walks two
                                   (4096, 4096, 64)])
def test_f32_tile_staging_variants_agree(device, monkeypatch, M, N, K):
    # fp32 products have a register-staged kernel and one whose tiles are copied straight into
    # LDS (K a multiple of 32); same tiles and k order, so the results must be identical bits
    # for the forward (k/k), dX (k/n) and dW (m/n) operand layouts, ragged tile edges included.
    x = normal(59, 0, (M, K))
    w = normal(59, 1, (N, K), std=0.05)
    b = normal(59, 2, (N,), std=0.1)
    dy = normal(59, 3, (M, N), std=0.5)
    # (an output of few tiles would be split along K, which changes the order of the sums:
    # switched off for the bitwise comparison, on again for the comparison with the oracle)
    monkeypatch.setenv("MOGRAD_HIP_GEMM_SPLITK_MIN_K", str(1 << 30))
    monkeypatch.setenv("MOGRAD_HIP_GEMM_F32_PIPE", "0")
    base = _linear_all(device, x, w, b, dy)
    monkeypatch.delenv("MOGRAD_HIP_GEMM_F32_PIPE")
    got = _linear_all(device, x, w, b, dy)
    for g, want, name in zip(got, base, ("y", "dx", "dw", "db")):
        np.testing.assert_array_equal(g, want, err_msg=name)
    monkeypatch.delenv("MOGRAD_HIP_GEMM_SPLITK_MIN_K")
    got = _linear_all(device, x, w, b, dy)
    assert_sum_close(got[0], O.matmul_bias_bt(x, w, b), np.abs(x) @ np.abs(w).T, what="y")
    assert_sum_close(got[1], O.linear_grad_x(dy, w), np.abs(dy) @ np.abs(w), what="dx")
    assert_sum_close(got[2], O.linear_grad_w(dy, x), np.abs(dy).T @ np.abs(x), what="dw")


@pytest.mark.parametrize("M,N,K", [(8192, 2048, 1024), (4104, 4000, 1088), (2048, 8192, 2048)])
def test_large_products_agree_with_the_register_staged_kernel(device, monkeypatch, M, N, K):
    # A product large enough that the library picks 256 x 256 tiles by itself (K >= 1024 and
    # a tile for every CU) must equal the register-staged kernel's result bit for bit, for
    # the forward and both gradient layouts, also with ragged last tiles in both directions.
    x = round_to_dtype(normal(58, 0, (M, K)), BF16)
    w = round_to_dtype(normal(58, 1, (N, K), std=0.05), BF16)
    dy = round_to_dtype(normal(58, 2, (M, N), std=0.5), BF16)
    lib, st = device.lib, device.stream
    bx, bw, bdy = (AnyBuffer.from_numpy(device, a, BF16) for a in (x, w, dy))

    def run():
        y, dx, dw = (AnyBuffer.create(BF16, device, n) for n in (M * N, M * K, N * K))
        lib.mg_matmul_bt(bx.data_ptr(), bw.data_ptr(), y.data_ptr(), 1, M, N, K, K, 1, K, 1, M * K, N * K, BF16, st)
        lib.mg_linear_bwd(bdy.data_ptr(), bx.data_ptr(), bw.data_ptr(), dx.data_ptr(), dw.data_ptr(), None, M, N, K, BF16, st)
        return y.to_numpy((M, N)), dx.to_numpy((M, K)), dw.to_numpy((N, K))

    auto = run()
    monkeypatch.setenv("MOGRAD_HIP_GEMM16_PIPE", "0")
    base = run()
    for got, want, name in zip(auto, base, ("y", "dx", "dw")):
        np.testing.assert_array_equal(got, want, err_msg=name)
    # and a spot check of the forward against float64 on a few rows
    rows = [0, 257, M // 2 - 1, M - 1]
    want = x[rows].astype(np.float64) @ w.astype(np.float64).T
    assert_close(auto[0][rows], want, 1.6e-2, 1.6e-2 * np.abs(want).max(), "y rows")


@pytest.mark.parametrize("variant", ["0", "322", "642", "2322", "2642"])
def test_batched_projections_tile_staging_variants(device, monkeypatch, variant):
    # The same two batched products (batch stride 0 on the shared operand; the second split
    # along K with the batch in the grid's z) through each 16-bit tile-staging variant.
    monkeypatch.setenv("MOGRAD_HIP_GEMM16_PIPE", variant)
    lib, st, dtype, M, d = device.lib, device.stream, BF16, 2048, 128
    x = round_to_dtype(normal(57, 0, (M, d)), dtype)
    w = round_to_dtype(normal(57, 1, (3, d, d), std=0.1), dtype)
    dy = round_to_dtype(normal(57, 2, (3, M, d), std=0.5), dtype)
    bx, bw, bdy = (AnyBuffer.from_numpy(device, a, dtype) for a in (x, w, dy))
    y, dw = AnyBuffer.create(dtype, device, 3 * M * d), AnyBuffer.create(dtype, device, 3 * d * d)
    lib.mg_matmul_bt(bx.data_ptr(), bw.data_ptr(), y.data_ptr(), 3, M, d, d, d, 1, d, 1, 0, d * d, dtype, st)
    lib.mg_matmul(bdy.data_ptr(), bx.data_ptr(), dw.data_ptr(), 3, d, d, M, 1, d, d, 1, M * d, 0, dtype, st)
    want_y = np.einsum("tk,bnk->btn", x.astype(np.float64), w.astype(np.float64))
    want_dw = np.einsum("bto,ti->boi", dy.astype(np.float64), x.astype(np.float64))
    assert_close(y.to_numpy((3, M, d)), want_y, 1.6e-2, 1.6e-2 * np.abs(want_y).max(), "y")
    assert_close(dw.to_numpy((3, d, d)), want_dw, 1.6e-2, 1.6e-2 * np.abs(want_dw).max(), "dw")


# ---- fused epilogues: each must give exactly what the separate calls give -----------------

FUSED_SHAPES = [(256, 384, 512), (200, 136, 264), (130, 65, 384), (64, 10, 256), (33, 7, 5), (4096, 128, 128),
                (128, 64, 4096), (256, 10, 2048)]


def _ptr(b):
    return b.data_ptr()


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("M,N,K", FUSED_SHAPES)
def test_fused_epilogues_equal_separate_calls(device, dtype, M, N, K):
    lib, st = device.lib, device.stream
    x = round_to_dtype(normal(49, 0, (M, K)), dtype)
    w = round_to_dtype(normal(49, 1, (N, K), std=0.1), dtype)
    b = round_to_dtype(normal(49, 2, (N,), std=0.5), dtype)
    res = round_to_dtype(normal(49, 3, (M, N)), dtype)
    dy = round_to_dtype(normal(49, 4, (M, N), std=0.5), dtype)
    bx, bw, bb, bres, bdy = (AnyBuffer.from_numpy(device, a, dtype) for a in (x, w, b, res, dy))
    new = lambda n: AnyBuffer.create(dtype, device, n)  # noqa: E731
    mm = (1, M, N, K, K, 1, K, 1, M * K, N * K, dtype, st)

    # A B^T + residual  ==  matmul_bt, then add
    y, y_ref, got = new(M * N), new(M * N), new(M * N)
    lib.mg_matmul_bt(_ptr(bx), _ptr(bw), _ptr(y), *mm)
    lib.mg_add(_ptr(y), _ptr(bres), _ptr(y_ref), M * N, dtype, st)
    lib.mg_matmul_bt_add(_ptr(bx), _ptr(bw), _ptr(bres), _ptr(got), *mm)
    np.testing.assert_array_equal(got.to_numpy(), y_ref.to_numpy())
    # in place: the residual buffer is also the destination
    inplace = AnyBuffer.from_numpy(device, res, dtype)
    lib.mg_matmul_bt_add(_ptr(bx), _ptr(bw), _ptr(inplace), _ptr(inplace), *mm)
    np.testing.assert_array_equal(inplace.to_numpy(), y_ref.to_numpy())
    # and against the oracle
    want = O.matmul_bias_bt(x, w) + res
    rt = {F32: 1e-4, F16: 2e-3, BF16: 1.6e-2}[dtype]
    assert_close(got.to_numpy((M, N)), want, rt, rt * np.abs(want).max(), "matmul_bt_add")

    # max(A B^T + bias, 0)  ==  matmul_bias_bt, then relu
    lib.mg_matmul_bias_bt(_ptr(bx), _ptr(bw), _ptr(bb), _ptr(y), *mm)
    lib.mg_relu(_ptr(y), _ptr(y_ref), M * N, dtype, st)
    lib.mg_matmul_bias_relu_bt(_ptr(bx), _ptr(bw), _ptr(bb), _ptr(got), *mm)
    np.testing.assert_array_equal(got.to_numpy(), y_ref.to_numpy())

    # linear_bwd_fused: relu mask from x, accumulation into dx
    xr = np.maximum(x, 0)  # x as the output of a relu: about half zeros
    bxr = AnyBuffer.from_numpy(device, xr, dtype)
    dx, dx_ref, dw, dw_ref, db, db_ref = new(M * K), new(M * K), new(N * K), new(N * K), new(N), new(N)
    lib.mg_linear_bwd(_ptr(bdy), _ptr(bxr), _ptr(bw), _ptr(dx), _ptr(dw_ref), _ptr(db_ref), M, N, K, dtype, st)
    lib.mg_relu_grad(_ptr(bxr), _ptr(dx), _ptr(dx_ref), M * K, dtype, st)
    lib.mg_linear_bwd_fused(_ptr(bdy), _ptr(bxr), _ptr(bw), _ptr(dx), _ptr(dw), _ptr(db), M, N, K, 0, 1, dtype, st)
    np.testing.assert_array_equal(dx.to_numpy(), dx_ref.to_numpy())
    np.testing.assert_array_equal(dw.to_numpy(), dw_ref.to_numpy())
    np.testing.assert_array_equal(db.to_numpy(), db_ref.to_numpy())
    assert not dx.to_numpy((M, K))[xr <= 0].any()
    # accumulate: dx starts as `prior`, ends as prior + dY W
    prior = round_to_dtype(normal(49, 5, (M, K)), dtype)
    acc = AnyBuffer.from_numpy(device, prior, dtype)
    bprior = AnyBuffer.from_numpy(device, prior, dtype)
    lib.mg_linear_bwd(_ptr(bdy), _ptr(bx), _ptr(bw), _ptr(dx), None, None, M, N, K, dtype, st)
    lib.mg_add(_ptr(dx), _ptr(bprior), _ptr(dx_ref), M * K, dtype, st)
    lib.mg_linear_bwd_fused(_ptr(bdy), _ptr(bx), _ptr(bw), _ptr(acc), None, None, M, N, K, 1, 0, dtype, st)
    np.testing.assert_array_equal(acc.to_numpy(), dx_ref.to_numpy())


@pytest.mark.parametrize("dtype,rtol", [(F16, 2e-3), (BF16, 1.6e-2)])
@pytest.mark.parametrize("M,N,K", [(2048, 384, 384), (4096, 1152, 384), (2048, 1536, 384), (4096, 384, 1536),
                                   (1056, 96, 200), (1024, 64, 72), (2048, 832, 768)])
def test_linear_bwd_one_launch_matches_two(device, monkeypatch, dtype, rtol, M, N, K):
    # dX and dW of a 16-bit layer whose dW is split along the rows go out as one launch
    # (workgroups of both products in one grid); MOGRAD_HIP_LINEAR_BWD_ONE_LAUNCH=0 keeps the
    # two launches.  Same tiles, same k order: no bit may differ, also with the relu mask and
    # with accumulation into dx, and at ragged tile edges (K = 200, 72).
    lib, st = device.lib, device.stream
    x = np.maximum(round_to_dtype(normal(52, 0, (M, K)), dtype), 0)
    w = round_to_dtype(normal(52, 1, (N, K), std=0.05), dtype)
    dy = round_to_dtype(normal(52, 2, (M, N), std=0.5), dtype)
    prior = round_to_dtype(normal(52, 3, (M, K)), dtype)
    bx, bw, bdy = (AnyBuffer.from_numpy(device, a, dtype) for a in (x, w, dy))
    results = {}
    # the common launch splits dW for one workgroup per CU; ask the separate launch for the same
    monkeypatch.setenv("MOGRAD_HIP_GEMM_SPLITK_WG_PER_CU", "1")
    # Input widths that are multiples of 384 take 128 x 384 tiles in the common launch, with dW's
    # K ranges cut differently: "wide" is compared within the tolerance, the 128 x 128 form bitwise.
    modes = ("0", "1", "wide") if K % 384 == 0 else ("0", "1")
    for mode in modes:
        monkeypatch.setenv("MOGRAD_HIP_LINEAR_BWD_ONE_LAUNCH", "0" if mode == "0" else "1")
        monkeypatch.setenv("MOGRAD_HIP_LINEAR_BWD_WIDE", "1" if mode == "wide" else "0")
        out = []
        for accumulate, masked in ((0, 0), (1, 1)):
            dx = AnyBuffer.from_numpy(device, prior, dtype)
            dw, db = AnyBuffer.create(dtype, device, N * K), AnyBuffer.create(dtype, device, N)
            lib.mg_linear_bwd_fused(_ptr(bdy), _ptr(bx), _ptr(bw), _ptr(dx), _ptr(dw), _ptr(db), M, N, K, accumulate,
                                    masked, dtype, st)
            out += [dx.to_numpy((M, K)), dw.to_numpy((N, K)), db.to_numpy()]
        results[mode] = out
    # Launched alone, a dX with fewer tiles than CUs and a long reduction is itself split along
    # N (fp32 partials, another summation order); inside the common launch it never is.
    dx_split_alone = -(-M // 128) * -(-K // 128) < 256 and N >= 1024
    # In the common launch the bias gradient comes from the dW workgroups' dY tiles, one partial
    # row per K range: another (fixed) summation order than mg_sum_axis on its own.
    for got, base, name in zip(results["1"], results["0"], ("dx", "dw", "db", "dx masked+acc", "dw'", "db'")):
        if (name.startswith("dx") and dx_split_alone) or name.startswith("db"):
            assert_close(got, base, rtol, rtol * np.abs(base).max(), name)
        else:
            np.testing.assert_array_equal(got, base, err_msg=name)
    want_db, want_dx, want_dw = O.linear_grad_b(dy), O.linear_grad_x(dy, w), O.linear_grad_w(dy, x)
    for mode in modes[1:]:
        res = results[mode]
        np.testing.assert_array_equal(res[2], res[5], err_msg="db, second call")
        np.testing.assert_array_equal(res[1], res[4], err_msg="dw, second call")
        assert_close(res[2], want_db, rtol, rtol * np.abs(want_db).max(), "db")
        for got, want, name in ((res[0], want_dx, "dx"), (res[1], want_dw, "dw")):
            assert_close(got, want, rtol, rtol * np.abs(want).max(), f"{name} ({mode})")
        assert_close(res[3], prior + want_dx * (x > 0), 2 * rtol, 2 * rtol * np.abs(want_dx).max(), "dx masked+acc")
    if "wide" in results:
        # same dX tiles' k order (one tile is three of the narrow ones side by side): bitwise
        if not dx_split_alone:
            np.testing.assert_array_equal(results["wide"][0], results["0"][0], err_msg="dx wide")
            np.testing.assert_array_equal(results["wide"][3], results["0"][3], err_msg="dx masked+acc wide")


@pytest.mark.parametrize("dtype,rtol", [(F16, 2e-3), (BF16, 1.6e-2)])
@pytest.mark.parametrize("M,N,K", [(4096, 65, 384), (1024, 72, 64), (2048, 100, 200), (1056, 33, 136)])
def test_linear_bwd_ragged_width(device, monkeypatch, dtype, rtol, M, N, K):
    # A width that is no multiple of 32 (the 65-symbol head): dY and W are zero-padded to the
    # next multiple inside the call and go through the common launch; without it
    # (MOGRAD_HIP_LINEAR_BWD_ONE_LAUNCH=0) the element-staged kernels take both products.
    # Both against the oracle; dX also bit for bit (the padding adds exact zeros, same k order).
    lib, st = device.lib, device.stream
    x = np.maximum(round_to_dtype(normal(53, 0, (M, K)), dtype), 0)
    w = round_to_dtype(normal(53, 1, (N, K), std=0.05), dtype)
    dy = round_to_dtype(normal(53, 2, (M, N), std=0.5), dtype)
    prior = round_to_dtype(normal(53, 3, (M, K)), dtype)
    bx, bw, bdy = (AnyBuffer.from_numpy(device, a, dtype) for a in (x, w, dy))
    results = {}
    for mode in ("0", "1"):
        monkeypatch.setenv("MOGRAD_HIP_LINEAR_BWD_ONE_LAUNCH", mode)
        dx = AnyBuffer.from_numpy(device, prior, dtype)
        # canaries behind dW: only N rows may be written although the padded product has more
        dw = AnyBuffer.from_numpy(device, np.full((N + 32) * K, 7.0, np.float32), dtype)
        db = AnyBuffer.create(dtype, device, N)
        lib.mg_linear_bwd_fused(_ptr(bdy), _ptr(bx), _ptr(bw), _ptr(dx), _ptr(dw), _ptr(db), M, N, K, 1, 1, dtype, st)
        dw_all = dw.to_numpy((N + 32, K))
        assert (dw_all[N:] == 7.0).all()
        results[mode] = (dx.to_numpy((M, K)), dw_all[:N], db.to_numpy())
    np.testing.assert_array_equal(results["1"][0], results["0"][0], err_msg="dx")
    np.testing.assert_array_equal(results["1"][2], results["0"][2], err_msg="db")
    want_dx = prior + O.linear_grad_x(dy, w) * (x > 0)
    want_dw = O.linear_grad_w(dy, x)
    for mode in ("0", "1"):
        assert_close(results[mode][0], want_dx, 2 * rtol, 2 * rtol * np.abs(want_dx).max(), "dx " + mode)
        assert_close(results[mode][1], want_dw, rtol, rtol * np.abs(want_dw).max(), "dw " + mode)


LN_CONT_SHAPES = [(4096, 1152, 384), (2048, 1536, 384), (2112, 768, 384), (16384, 1536, 384),  # one launch, whole rows
                  (1024, 384, 384), (512, 96, 200), (2048, 832, 768)]                              # separate kernels


# fp32 always takes the two separate entries: the largest shapes add nothing there
LN_CONT_CASES = [(dt, *shape) for dt in (BF16, F16, F32) for shape in LN_CONT_SHAPES
                 if dt != F32 or shape[0] * shape[1] * shape[2] <= 2048 * 1536 * 384]


@pytest.mark.parametrize("deferred", [False, True])
@pytest.mark.parametrize("dtype,M,N,K", LN_CONT_CASES)
def test_linear_bwd_continues_as_layer_norm_bwd(device, dtype, M, N, K, deferred):
    # Y = LN(h) W^T + b: the layer's backward and the LayerNorm's in one entry.  For 16-bit layers
    # of 384 input columns the dX tiles hold whole rows and finish as the LayerNorm backward
    # inside the launch ((2112, ..): the last tile is half empty); other shapes and fp32 run the
    # two separate entries on a scratch tensor.  Either way dW and db are the separate entry's
    # bits, and dh, dgamma and dbeta differ from the separate calls only by the order of their
    # fp32 sums; the oracle gets the same dY W rounded to the tensors' type.
    lib, st = device.lib, device.stream
    h = round_to_dtype(normal(81, 0, (M, K), std=1.5) + 0.3, dtype)
    gamma = round_to_dtype(uniform(81, 1, (K,), 0.5, 1.5), dtype)
    beta = round_to_dtype(normal(81, 2, (K,), std=0.1), dtype)
    w = round_to_dtype(normal(81, 3, (N, K), std=0.1), dtype)
    dy = round_to_dtype(normal(81, 4, (M, N), std=0.5), dtype)
    prior = round_to_dtype(normal(81, 5, (M, K)), dtype)
    bh, bg, bbeta, bw, bdy, bprior = (AnyBuffer.from_numpy(device, a, dtype) for a in (h, gamma, beta, w, dy, prior))
    new = lambda n, dt=dtype: AnyBuffer.create(dt, device, n)  # noqa: E731
    x, mean, rstd = new(M * K), new(M, F32), new(M, F32)
    lib.mg_layer_norm_fwd_stats(_ptr(bh), _ptr(bg), _ptr(bbeta), _ptr(x), _ptr(mean), _ptr(rstd), M, K, 1e-5, dtype, st)
    # the two separate entries
    t, dh_ref, dw_ref, db_ref, dg_ref, dbt_ref = new(M * K), new(M * K), new(N * K), new(N), new(K), new(K)
    lib.mg_linear_bwd(_ptr(bdy), _ptr(x), _ptr(bw), _ptr(t), _ptr(dw_ref), _ptr(db_ref), M, N, K, dtype, st)
    lib.mg_layer_norm_bwd_stats_add(_ptr(t), _ptr(bh), _ptr(bg), _ptr(mean), _ptr(rstd), _ptr(bprior), _ptr(dh_ref),
                                    _ptr(dg_ref), _ptr(dbt_ref), M, K, dtype, st)
    # the one entry, dh in place on top of the prior gradient
    gdt = F32 if deferred else dtype
    dh = AnyBuffer.from_numpy(device, prior, dtype)
    dw, db, dg, dbt = new(N * K, gdt), new(N, gdt), new(K, gdt), new(K, gdt)
    pending = C.c_void_p()
    if deferred:
        lib.mg_deferred_create(C.byref(pending))
    try:
        lib.mg_linear_bwd_layer_norm_bwd(_ptr(bdy), _ptr(x), _ptr(bw), _ptr(bh), _ptr(bg), _ptr(mean), _ptr(rstd), _ptr(dh),
                                         _ptr(dw), _ptr(db), _ptr(dg), _ptr(dbt), M, N, K, 1, dtype, gdt,
                                         pending if deferred else None, st)
        if deferred:
            lib.mg_finish_deferred(pending, st)
    finally:
        if deferred:
            lib.mg_deferred_destroy(pending)
    ulp = {F32: 2.0 ** -21, F16: 2.0 ** -9, BF16: 2.0 ** -6}[dtype]  # two units in the last place
    if deferred:  # fp32 sums before the rounding of the immediate forms
        np.testing.assert_array_equal(round_to_dtype(dw.to_numpy(), dtype), dw_ref.to_numpy())
        np.testing.assert_array_equal(round_to_dtype(db.to_numpy(), dtype), db_ref.to_numpy())
    else:
        np.testing.assert_array_equal(dw.to_numpy(), dw_ref.to_numpy())
        np.testing.assert_array_equal(db.to_numpy(), db_ref.to_numpy())
    got, ref = dh.to_numpy((M, K)).astype(np.float64), dh_ref.to_numpy((M, K)).astype(np.float64)
    # (the gradient is rounded before the prior is added: a unit in its last place, not the sum's)
    assert np.all(np.abs(got - ref) <= ulp * (np.abs(ref) + np.abs(prior)) + 1e-5 * np.abs(ref).max())
    assert np.mean(got == ref) > 0.98
    tv = t.to_numpy((M, K)).astype(np.float64)
    for g_, r_, mass in ((dg, dg_ref, np.abs(tv).sum(axis=0) * 4.0), (dbt, dbt_ref, np.abs(tv).sum(axis=0))):
        gv, rv = g_.to_numpy().astype(np.float64), r_.to_numpy().astype(np.float64)
        assert np.all(np.abs(gv - rv) <= ulp * np.abs(rv) + 2.0 ** -20 * mass)
    if M <= 4096:  # and the oracle, from the rounded dY W the kernels saw
        odx, odg, odb = O.layer_norm_bwd(tv, h, gamma)
        rt = {F32: 1e-4, F16: 2e-3, BF16: 1.6e-2}[dtype]
        assert_close(got, round_to_dtype(odx, dtype).astype(np.float64) + prior, rt, rt * np.abs(odx).max(), "dh")
        assert_close(dg.to_numpy(), odg, rt, rt * np.abs(odg).max(), "dgamma")
        assert_close(dbt.to_numpy(), odb, rt, rt * np.abs(odb).max(), "dbeta")


@pytest.mark.parametrize("M,N,K", [(2048, 1152, 384), (1024, 384, 384)])
def test_linear_bwd_layer_norm_bwd_without_prior_and_bias(device, M, N, K):
    # dx_accumulate = 0 (dh is written, whatever it held) and db = NULL, in the one launch and in
    # the separate-kernels form.
    dtype = BF16
    lib, st = device.lib, device.stream
    h = round_to_dtype(normal(82, 0, (M, K), std=2.0), dtype)
    gamma = round_to_dtype(uniform(82, 1, (K,), 0.5, 1.5), dtype)
    w = round_to_dtype(normal(82, 3, (N, K), std=0.1), dtype)
    dy = round_to_dtype(normal(82, 4, (M, N), std=0.5), dtype)
    bh, bg, bw, bdy = (AnyBuffer.from_numpy(device, a, dtype) for a in (h, gamma, w, dy))
    new = lambda n, dt=dtype: AnyBuffer.create(dt, device, n)  # noqa: E731
    x, mean, rstd = new(M * K), new(M, F32), new(M, F32)
    lib.mg_layer_norm_fwd_stats(_ptr(bh), _ptr(bg), _ptr(bg), _ptr(x), _ptr(mean), _ptr(rstd), M, K, 1e-5, dtype, st)
    t, dh_ref, dw_ref, dg_ref, dbt_ref = new(M * K), new(M * K), new(N * K), new(K), new(K)
    lib.mg_linear_bwd(_ptr(bdy), _ptr(x), _ptr(bw), _ptr(t), _ptr(dw_ref), None, M, N, K, dtype, st)
    lib.mg_layer_norm_bwd_stats(_ptr(t), _ptr(bh), _ptr(bg), _ptr(mean), _ptr(rstd), _ptr(dh_ref), _ptr(dg_ref),
                                _ptr(dbt_ref), M, K, dtype, st)
    dh = AnyBuffer.create(dtype, device, M * K, fill=123.0)  # must be overwritten, not added to
    dw, dg, dbt = new(N * K), new(K), new(K)
    lib.mg_linear_bwd_layer_norm_bwd(_ptr(bdy), _ptr(x), _ptr(bw), _ptr(bh), _ptr(bg), _ptr(mean), _ptr(rstd), _ptr(dh),
                                     _ptr(dw), None, _ptr(dg), _ptr(dbt), M, N, K, 0, dtype, dtype, None, st)
    np.testing.assert_array_equal(dw.to_numpy(), dw_ref.to_numpy())
    got, ref = dh.to_numpy().astype(np.float64), dh_ref.to_numpy().astype(np.float64)
    assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 1e-5 * np.abs(ref).max()) and np.mean(got == ref) > 0.98
    for g_, r_ in ((dg, dg_ref), (dbt, dbt_ref)):
        gv, rv = g_.to_numpy().astype(np.float64), r_.to_numpy().astype(np.float64)
        assert np.all(np.abs(gv - rv) <= 2.0 ** -6 * np.abs(rv) + 1e-3 * np.abs(rv).max())
    with pytest.raises(MogradError):  # dgamma is not optional
        lib.mg_linear_bwd_layer_norm_bwd(_ptr(bdy), _ptr(x), _ptr(bw), _ptr(bh), _ptr(bg), _ptr(mean), _ptr(rstd), _ptr(dh),
                                         _ptr(dw), None, None, _ptr(dbt), M, N, K, 0, dtype, dtype, None, st)
    with pytest.raises(MogradError):  # without a list the gradients have the tensors' type
        lib.mg_linear_bwd_layer_norm_bwd(_ptr(bdy), _ptr(x), _ptr(bw), _ptr(bh), _ptr(bg), _ptr(mean), _ptr(rstd), _ptr(dh),
                                         _ptr(dw), None, _ptr(dg), _ptr(dbt), M, N, K, 0, dtype, F32, None, st)


@pytest.mark.parametrize("M,N,acc", [(0, 64, 1), (128, 0, 1), (128, 0, 0)])
def test_linear_bwd_layer_norm_bwd_empty_sides(device, M, N, acc):
    # No rows: every sum is zero and dh is left alone.  No output features: dY W is zero, so dh
    # keeps its prior (or becomes zero), and the LayerNorm's sums are zero.
    dtype, K = BF16, 384
    lib, st = device.lib, device.stream
    new = lambda n, fill, dt=dtype: AnyBuffer.create(dt, device, max(n, 1), fill=fill)  # noqa: E731
    dy, x, w, h, g = new(M * N, 0.5), new(M * K, 0.25), new(N * K, 0.125), new(M * K, 1.0), new(K, 1.0)
    mean, rstd = new(M, 0.0, F32), new(M, 1.0, F32)
    dh, dw, db, dg, dbt = new(M * K, 3.0), new(N * K, 7.0), new(N, 7.0), new(K, 7.0), new(K, 7.0)
    lib.mg_linear_bwd_layer_norm_bwd(_ptr(dy), _ptr(x), _ptr(w), _ptr(h), _ptr(g), _ptr(mean), _ptr(rstd), _ptr(dh),
                                     _ptr(dw), _ptr(db), _ptr(dg), _ptr(dbt), M, N, K, acc, dtype, dtype, None, st)
    assert np.all(dg.to_numpy() == 0) and np.all(dbt.to_numpy() == 0)
    if M:
        assert np.all(dh.to_numpy() == (3.0 if acc else 0.0))
    if N:
        assert np.all(dw.to_numpy() == 0) and np.all(db.to_numpy() == 0)


def test_fused_entry_errors(device):
    buf = AnyBuffer.create(F32, device, 16)
    p = buf.data_ptr()
    with pytest.raises(MogradError, match="null residual"):
        device.lib.mg_matmul_bt_add(p, p, None, p, 1, 2, 2, 2, 2, 1, 2, 1, 4, 4, F32, device.stream)
    with pytest.raises(MogradError, match="null bias"):
        device.lib.mg_matmul_bias_relu_bt(p, p, None, p, 1, 2, 2, 2, 2, 1, 2, 1, 4, 4, F32, device.stream)
    with pytest.raises(MogradError, match="relu mask"):
        device.lib.mg_linear_bwd_fused(p, None, p, p, None, None, 2, 2, 2, 0, 1, F32, device.stream)
