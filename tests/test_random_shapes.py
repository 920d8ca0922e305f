"""Seeded sweeps over odd shapes: every case is small enough for the float64 oracle, and
the point is the dispatch (aligned / ragged / split-K / generic GEMM paths, attention tile
edges, row-kernel shape ladders), not the size."""
import math

import numpy as np
import pytest

from helpers import ATOL_F32, RTOL_F32, assert_close
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu

from mograd_amd import BF16, F16, F32, I32, AnyBuffer, Layout, Node  # noqa: E402
from mograd_amd import runtime as R  # noqa: E402
from mograd_amd.runtime import round_to_dtype  # noqa: E402

RT = {F32: 2e-4, F16: 2e-3, BF16: 1.6e-2}


def test_random_linear_shapes(device):
    rng = np.random.Generator(np.random.PCG64(95_000))
    lib, st = device.lib, device.stream
    for case in range(60):
        dtype = (F32, F16, BF16)[case % 3]
        M, N, K = (int(v) for v in rng.integers(1, 300, 3))
        if case % 5 == 0:
            K = int(rng.integers(1024, 3000))  # long reductions: split-K for the small outputs
        x = round_to_dtype(rng.standard_normal((M, K)).astype(np.float32), dtype)
        w = round_to_dtype((rng.standard_normal((N, K)) * 0.1).astype(np.float32), dtype)
        b = round_to_dtype(rng.standard_normal(N).astype(np.float32), dtype)
        dy = round_to_dtype(rng.standard_normal((M, N)).astype(np.float32), dtype)
        bx, bw, bb, bdy = (AnyBuffer.from_numpy(device, a, dtype) for a in (x, w, b, dy))
        y, dx, dw, db = (AnyBuffer.create(dtype, device, n) for n in (M * N, M * K, N * K, N))
        lib.mg_matmul_bias_bt(bx.data_ptr(), bw.data_ptr(), bb.data_ptr(), y.data_ptr(), 1, M, N, K, K, 1, K, 1, M * K,
                              N * K, dtype, st)
        lib.mg_linear_bwd(bdy.data_ptr(), bx.data_ptr(), bw.data_ptr(), dx.data_ptr(), dw.data_ptr(), db.data_ptr(), M, N,
                          K, dtype, st)
        rt = RT[dtype]
        for got, want, name in ((y.to_numpy((M, N)), O.matmul_bias_bt(x, w, b), "y"),
                                (dx.to_numpy((M, K)), O.linear_grad_x(dy, w), "dx"),
                                (dw.to_numpy((N, K)), O.linear_grad_w(dy, x), "dw"),
                                (db.to_numpy(), O.linear_grad_b(dy), "db")):
            assert_close(got, want, rt, rt * max(np.abs(want).max(), 1e-3), f"case {case} {(M, N, K)} dtype {dtype} {name}")


def test_random_thin_f32_products(device):
    # fp32 heads of a few classes behind wide layers: the forward has fewer output tiles than
    # the device has CUs (split along K when K is a multiple of 32 and at least 1024), and
    # dW = dY^T X reads the (M, N) gradient along its N-wide rows (copied k-contiguous when
    # M is a multiple of 4 and at least 512); neighbouring shapes take the other paths
    rng = np.random.Generator(np.random.PCG64(95_300))
    lib, st = device.lib, device.stream
    for case in range(16):
        N = int(rng.integers(1, 21))
        M = int(rng.integers(128, 513)) * 4 if case % 4 != 3 else int(rng.integers(500, 2050))
        K = int(rng.integers(8, 97)) * 32 if case % 4 != 2 else int(rng.integers(256, 3000))
        x = rng.standard_normal((M, K)).astype(np.float32)
        w = (rng.standard_normal((N, K)) * 0.1).astype(np.float32)
        b = rng.standard_normal(N).astype(np.float32)
        dy = rng.standard_normal((M, N)).astype(np.float32)
        bx, bw, bb, bdy = (AnyBuffer.from_numpy(device, a, F32) for a in (x, w, b, dy))
        y, dx, dw, db = (AnyBuffer.create(F32, device, n) for n in (M * N, M * K, N * K, N))
        lib.mg_matmul_bias_bt(bx.data_ptr(), bw.data_ptr(), bb.data_ptr(), y.data_ptr(), 1, M, N, K, K, 1, K, 1, M * K,
                              N * K, F32, st)
        lib.mg_linear_bwd(bdy.data_ptr(), bx.data_ptr(), bw.data_ptr(), dx.data_ptr(), dw.data_ptr(), db.data_ptr(), M, N,
                          K, F32, st)
        rt = RT[F32]
        for got, want, name in ((y.to_numpy((M, N)), O.matmul_bias_bt(x, w, b), "y"),
                                (dx.to_numpy((M, K)), O.linear_grad_x(dy, w), "dx"),
                                (dw.to_numpy((N, K)), O.linear_grad_w(dy, x), "dw"),
                                (db.to_numpy(), O.linear_grad_b(dy), "db")):
            assert_close(got, want, rt, rt * max(np.abs(want).max(), 1e-3), f"case {case} {(M, N, K)} {name}")


def test_random_16bit_tile_staging_shapes(device, monkeypatch):
    # Shapes the LDS-copy GEMM kernels take (extents multiples of 8, K a multiple of 64), with
    # padded leading dimensions and batches, through every forced variant: all must equal the
    # register-staged kernel bit for bit, and that one the float64 product.
    rng = np.random.Generator(np.random.PCG64(95_100))
    lib, st = device.lib, device.stream
    for case in range(24):
        dtype = (F16, BF16)[case % 2]
        batch = int(rng.integers(1, 4))
        M, N = (8 * int(v) for v in rng.integers(1, 66, 2))
        K = 64 * int(rng.integers(1, 33 if case % 4 else 5))
        lda, ldb = K + 8 * int(rng.integers(0, 3)), K + 8 * int(rng.integers(0, 3))
        a = round_to_dtype(rng.standard_normal((batch, M, lda)).astype(np.float32), dtype)
        b = round_to_dtype((rng.standard_normal((batch, N, ldb)) * 0.1).astype(np.float32), dtype)
        ba, bb = AnyBuffer.from_numpy(device, a, dtype), AnyBuffer.from_numpy(device, b, dtype)
        results = {}
        for variant in ("0", "322", "642", "2322", "2642"):
            monkeypatch.setenv("MOGRAD_HIP_GEMM16_PIPE", variant)
            nt, nn, tn = (AnyBuffer.create(dtype, device, n) for n in (batch * M * N, batch * M * ldb, batch * lda * N))
            # C = A B^T over k (both k-contiguous)
            lib.mg_matmul_bt(ba.data_ptr(), bb.data_ptr(), nt.data_ptr(), batch, M, N, K, lda, 1, ldb, 1, M * lda, N * ldb,
                             dtype, st)
            # C2(M, ldb) = C(M, N) B(N, ldb): right operand n-contiguous (the dX layout); K here is N
            # C3(lda, N) = A^T(lda, M) C(M, N): left operand m-contiguous (the dW layout); K here is M
            if N % 64 == 0:
                lib.mg_matmul(nt.data_ptr(), bb.data_ptr(), nn.data_ptr(), batch, M, ldb, N, N, 1, ldb, 1, M * N, N * ldb,
                              dtype, st)
            if M % 64 == 0:
                lib.mg_matmul(ba.data_ptr(), nt.data_ptr(), tn.data_ptr(), batch, lda, N, M, 1, lda, N, 1, M * lda, M * N,
                              dtype, st)
            results[variant] = (nt.to_numpy((batch, M, N)), nn.to_numpy((batch, M, ldb)) if N % 64 == 0 else None,
                                tn.to_numpy((batch, lda, N)) if M % 64 == 0 else None)
        what = f"case {case} batch {batch} {(M, N, K)} ld {(lda, ldb)} dtype {dtype}"
        for variant in ("322", "642", "2322", "2642"):
            for got, base, name in zip(results[variant], results["0"], ("nt", "nn", "tn")):
                if base is not None:
                    np.testing.assert_array_equal(got, base, err_msg=f"{what} {name} variant {variant}")
        want = np.einsum("bmk,bnk->bmn", a[:, :, :K].astype(np.float64), b[:, :, :K].astype(np.float64))
        rt = RT[dtype]
        assert_close(results["0"][0], want, rt, rt * max(np.abs(want).max(), 1e-3), what)
    monkeypatch.delenv("MOGRAD_HIP_GEMM16_PIPE")


def test_random_attention_shapes(device):
    rng = np.random.Generator(np.random.PCG64(96_000))
    lib, st = device.lib, device.stream
    for case in range(24):
        dtype = (BF16, F16)[case % 2]
        B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
        S = int(rng.integers(1, 300))
        D = int(rng.integers(1, 17)) * 8
        causal = case % 3 == 0
        scale = 1.0 / math.sqrt(D)
        q, k, v = (round_to_dtype(rng.standard_normal((B, S, H, D)).astype(np.float32), dtype) for _ in range(3))
        do = round_to_dtype(rng.standard_normal((B, H, S, D)).astype(np.float32), dtype)
        bq, bk, bv, bdo = (AnyBuffer.from_numpy(device, a, dtype) for a in (q, k, v, do))
        n = B * S * H * D
        o, dq, dk, dv = (AnyBuffer.create(dtype, device, n) for _ in range(4))
        lse = AnyBuffer.create(F32, device, B * H * S)
        lib.mg_flash_attn_fwd(bq.data_ptr(), bk.data_ptr(), bv.data_ptr(), None, o.data_ptr(), lse.data_ptr(), B, S, H, D,
                              scale, int(causal), 0, dtype, st)
        lib.mg_flash_attn_bwd(bdo.data_ptr(), o.data_ptr(), bq.data_ptr(), bk.data_ptr(), bv.data_ptr(), None,
                              lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, S, H, D, scale, int(causal),
                              0, dtype, st)
        wo, wl = O.sdpa_fwd(q, k, v, None, causal, scale)
        wdq, wdk, wdv = O.sdpa_bwd(q, k, v, do, None, causal, scale)
        tol = 2e-2 if dtype == BF16 else 4e-3
        what = f"case {case} B{B} S{S} H{H} D{D} causal={causal} dtype {dtype}"
        assert_close(lse.to_numpy((B, H, S)), wl, 1e-3, 2e-2 if dtype == BF16 else 4e-3, what + " lse")
        for got, want, name in ((o.to_numpy((B, H, S, D)), wo, "o"), (dq.to_numpy((B, S, H, D)), wdq, "dq"),
                                (dk.to_numpy((B, S, H, D)), wdk, "dk"), (dv.to_numpy((B, S, H, D)), wdv, "dv")):
            assert_close(got, want, tol, tol * max(np.abs(want).max(), 1e-3), what + " " + name)


def test_random_f32_attention_shapes(device):
    # fp32 tensors: head dims 1-160 (the matrix-core kernels for 32, 64 and 128 columns, element-wise
    # loads when D is not a multiple of four, the row-per-thread kernels above 128), lengths on both
    # sides of the 64-token threshold, every mask mode; the reference's widest fp32 budget for these
    # head dims (tests/kernels/attention/generic.mojo:440-665) against the f64 oracle.
    rng = np.random.Generator(np.random.PCG64(98_000))
    lib, st = device.lib, device.stream
    for case in range(24):
        B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
        S = int(rng.integers(1, 400))
        D = int(rng.integers(1, 161))
        causal, with_mask = case % 3 == 0, case % 3 == 1
        scale = 1.0 / math.sqrt(D)
        q, k, v = (rng.standard_normal((B, S, H, D)).astype(np.float32) for _ in range(3))
        do = rng.standard_normal((B, H, S, D)).astype(np.float32)
        m = rng.standard_normal((B, H, S, S)).astype(np.float32) if with_mask else None
        bq, bk, bv, bdo = (AnyBuffer.from_numpy(device, a, F32) for a in (q, k, v, do))
        bm = AnyBuffer.from_numpy(device, m, F32) if with_mask else None
        pm = bm.data_ptr() if with_mask else None
        n = B * S * H * D
        o, dq, dk, dv = (AnyBuffer.create(F32, device, n) for _ in range(4))
        lse = AnyBuffer.create(F32, device, B * H * S)
        lib.mg_flash_attn_fwd(bq.data_ptr(), bk.data_ptr(), bv.data_ptr(), pm, o.data_ptr(), lse.data_ptr(), B, S, H, D,
                              scale, int(causal), int(with_mask), F32, st)
        lib.mg_flash_attn_bwd(bdo.data_ptr(), o.data_ptr(), bq.data_ptr(), bk.data_ptr(), bv.data_ptr(), pm,
                              lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, S, H, D, scale, int(causal),
                              int(with_mask), F32, st)
        wo, wl = O.sdpa_fwd(q, k, v, m, causal, scale)
        wdq, wdk, wdv = O.sdpa_bwd(q, k, v, do, m, causal, scale)
        what = f"case {case} B{B} S{S} H{H} D{D} causal={causal} bias={with_mask}"
        for got, want, name in ((lse.to_numpy((B, H, S)), wl, "lse"), (o.to_numpy((B, H, S, D)), wo, "o"),
                                (dq.to_numpy((B, S, H, D)), wdq, "dq"), (dk.to_numpy((B, S, H, D)), wdk, "dk"),
                                (dv.to_numpy((B, S, H, D)), wdv, "dv")):
            err = float(np.max(np.abs(got.astype(np.float64) - want)))
            assert np.all(np.isfinite(got)) and err <= 2e-5, f"{what} {name}: {err}"


def _random_view(rng, shape):
    """Strides (elements), base offset and backing size of a random view of `shape`: the dims laid
    out in a random order, some broadcast (stride 0), some with a gap after them or every other
    element taken."""
    rank = len(shape)
    order = list(rng.permutation(rank))
    strides = [0] * rank
    step = int(rng.integers(1, 3))  # innermost memory dim: every element or every other
    for d in order:
        if shape[d] > 1 and rng.random() < 0.2:
            strides[d] = 0  # broadcast
            continue
        strides[d] = step
        step = step * shape[d] + int(rng.integers(0, 3)) * (rng.random() < 0.3)
    offset = int(rng.integers(0, 5))
    size = offset + 1 + sum((n - 1) * t for n, t in zip(shape, strides))
    return strides, offset, size


def test_random_strided_views(device):
    # add, relu, relu_grad, cast and softmax over random views of rank 1-5 (permuted, broadcast, gapped,
    # strided, offset), bit for bit against numpy on the same views (softmax: the oracle at the storage
    # type's rounding): the merging of dims and the choice of 16-byte accesses must never change a value.
    rng = np.random.Generator(np.random.PCG64(99_000))
    for case in range(60):
        dtype = (F32, BF16, F16)[case % 3]
        rank = int(rng.integers(1, 6))
        shape = [int(rng.choice([1, 2, 3, 4, 8, 16, 24, 32])) for _ in range(rank)]
        if case % 4 == 0:
            shape[-1] = int(rng.choice([8, 16, 64]))  # rows that can be read 16 bytes at a time
        (sa, oa, na), (sb, ob, nb) = _random_view(rng, shape), _random_view(rng, shape)
        if case % 5 == 0:
            sa, oa, na = list(Layout(*shape).stride()), 0, int(np.prod(shape))  # one operand plain
        a = round_to_dtype(rng.standard_normal(na).astype(np.float32), dtype)
        b = round_to_dtype(rng.standard_normal(nb).astype(np.float32), dtype)
        item = a.itemsize
        va = np.lib.stride_tricks.as_strided(a[oa:], shape, tuple(t * item for t in sa))
        vb = np.lib.stride_tricks.as_strided(b[ob:], shape, tuple(t * item for t in sb))
        la, lb = Layout(*shape, strides=sa, base_offset=oa), Layout(*shape, strides=sb, base_offset=ob)
        out = Layout(*shape)
        what = f"case {case} shape {shape} a {sa}+{oa} b {sb}+{ob} dtype {dtype}"

        def run(op, operands, to=dtype):
            srcs = [Node.leaf(l, d) for _, l, d in operands]
            bufs = [AnyBuffer.from_numpy(device, h, d).view(l) for h, l, d in operands]
            (res,) = R.run(Node(op, out, to, srcs, {}), bufs, device)
            return res.to_numpy(tuple(shape))

        np.testing.assert_array_equal(run("ADD", [(a, la, dtype), (b, lb, dtype)]), round_to_dtype(va + vb, dtype), what)
        np.testing.assert_array_equal(run("RELU_GRAD", [(a, la, dtype), (b, lb, dtype)]),
                                      np.where(va > 0, vb, 0).astype(np.float32), what)
        np.testing.assert_array_equal(run("RELU", [(a, la, dtype)]), np.maximum(va, 0), what)
        np.testing.assert_array_equal(run("CONTIGUOUS", [(b, lb, dtype)]), vb, what)
        to = (BF16, F32, F16)[case % 3]
        np.testing.assert_array_equal(run("CAST", [(a, la, dtype)], to), round_to_dtype(va, to), what)
        tol = {F32: 2e-6, F16: 1e-3, BF16: 8e-3}[dtype]
        np.testing.assert_allclose(run("SOFTMAX", [(a, la, dtype)]), O.softmax(va.astype(np.float64)), rtol=tol, atol=tol,
                                   err_msg=what)


def test_random_row_kernel_shapes(device):
    rng = np.random.Generator(np.random.PCG64(97_000))
    lib, st = device.lib, device.stream
    for case in range(40):
        rows = int(rng.integers(1, 70))
        cols = int(rng.choice([1, 3, 8, 17, 64, 100, 256, 257, 1000, 1024, 2052, 4100, 9000]))
        x = rng.standard_normal((rows, cols)).astype(np.float32) * 2 + 0.5
        dy = rng.standard_normal((rows, cols)).astype(np.float32)
        g = rng.uniform(0.5, 1.5, cols).astype(np.float32)
        bx, bdy, bg = (AnyBuffer.from_numpy(device, a) for a in (x, dy, g))
        dx, dg, db = (AnyBuffer.create(F32, device, n) for n in (rows * cols, cols, cols))
        lib.mg_layer_norm_bwd(bdy.data_ptr(), bx.data_ptr(), bg.data_ptr(), dx.data_ptr(), dg.data_ptr(), db.data_ptr(),
                              rows, cols, 1e-5, F32, st)
        wdx, wdg, wdb = O.layer_norm_bwd(dy, x, g, 1e-5)
        what = f"case {case} ({rows},{cols})"
        # narrow rows have a large 1/sqrt(var + eps): hold dx to the gradient's own scale
        assert_close(dx.to_numpy((rows, cols)), wdx, RTOL_F32, max(ATOL_F32, 1e-4 * np.abs(wdx).max()), what + " dx")
        assert_close(dg.to_numpy(), wdg, RTOL_F32, max(ATOL_F32, 1e-5 * np.abs(dy).sum(0).max() * np.abs(wdg).max() / max(np.abs(wdg).max(), 1)), what + " dgamma")
        assert_close(db.to_numpy(), wdb, RTOL_F32, max(ATOL_F32, 2e-6 * np.abs(dy).sum(0).max()), what + " dbeta")
        ids = rng.integers(0, cols, rows).astype(np.int32)
        bids = AnyBuffer.from_numpy(device, ids)
        loss, dl = AnyBuffer.create(F32, device, 1), AnyBuffer.create(F32, device, rows * cols)
        lib.mg_cross_entropy_fused_ids(bx.data_ptr(), bids.data_ptr(), None, loss.data_ptr(), dl.data_ptr(), rows, cols,
                                       F32, I32, st)
        assert_close(loss.item(), O.cross_entropy_ids(x, ids), RTOL_F32, ATOL_F32, what + " loss")
        assert_close(dl.to_numpy((rows, cols)), O.cross_entropy_grad_ids(x, ids), RTOL_F32, RTOL_F32 / rows, what + " dlogits")
