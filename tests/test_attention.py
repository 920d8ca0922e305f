"""Flash attention forward/backward on the GPU against the float64 oracle.

Follows the reference's attention tests: the f64 oracle and error budgets of
tests/kernels/attention/{harness,generic,mma}.mojo, the closed forms of
tests/test_ops.mojo:903-946 and tests/test_grad.mojo:1001-1023, through the same
dispatch surface (FLASH_ATTN / FLASH_ATTN_GRAD nodes).
"""
import math

import numpy as np
import pytest

from helpers import ATTN_BF16_FLOOR, RTOL_BF16_ATTN, assert_attn_grad_close, normal
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu

from mograd_amd import BF16, F16, F32, AnyBuffer, Layout, MogradError, Node  # noqa: E402
from mograd_amd import runtime as R  # noqa: E402
from mograd_amd.runtime import round_to_dtype  # noqa: E402


def _fwd(device, q, k, v, mask, causal, scale, dtype, mask_offset=0):
    B, S, H, D = q.shape
    attrs = {"scale": scale, "is_causal": causal, "has_bias": mask is not None}
    m = mask if mask is not None else np.zeros(8, np.float32)  # placeholder the kernels never read
    srcs = [Node.leaf(Layout(B, S, H, D), dtype)] * 3 + [Node.leaf(Layout(*m.shape), dtype)]
    node = Node("FLASH_ATTN", Layout(B, H, S, D), dtype, srcs, attrs)
    bufs = [AnyBuffer.from_numpy(device, a, dtype) for a in (q, k, v, m)]
    if mask_offset:  # the same bias, `mask_offset` elements into a larger allocation
        padded = np.concatenate([np.zeros(mask_offset, m.dtype), m.ravel()])
        bufs[3] = AnyBuffer.from_numpy(device, padded, dtype).view(Layout(m.size, base_offset=mask_offset))
    o, lse = R.run(node, bufs, device)
    return o, lse, bufs


def _fwd_bwd(device, q, k, v, do, mask=None, causal=False, scale=None, dtype=F32, mask_offset=0):
    """Forward for O/LSE chained into the backward, as the reference's run_bwd does
    (tests/kernels/attention/harness.mojo:266-344)."""
    B, S, H, D = q.shape
    scale = scale if scale is not None else 1.0 / math.sqrt(D)
    o, lse, (bq, bk, bv, bm) = _fwd(device, q, k, v, mask, causal, scale, dtype, mask_offset)
    attrs = {"scale": scale, "is_causal": causal, "has_bias": mask is not None}
    leaf = Node.leaf(Layout(B, S, H, D), dtype)
    srcs = [Node.leaf(Layout(B, H, S, D), dtype), Node.leaf(Layout(B, H, S, D), dtype), leaf, leaf, leaf,
            Node.leaf(Layout(bm.numel), dtype), Node.leaf(Layout(B, H, S), F32)]
    node = Node("FLASH_ATTN_GRAD", Layout(B, S, H, D), dtype, srcs, attrs)
    bdo = AnyBuffer.from_numpy(device, do, dtype)
    dq, dk, dv = R.run(node, [bdo, o, bq, bk, bv, bm, lse], device)
    return (o.to_numpy((B, H, S, D)), lse.to_numpy((B, H, S)), dq.to_numpy((B, S, H, D)), dk.to_numpy((B, S, H, D)),
            dv.to_numpy((B, S, H, D)))


def _inputs(cfg, B, S, H, D, dtype, with_mask):
    q, k, v = (round_to_dtype(normal(cfg, i, (B, S, H, D)), dtype) for i in range(3))
    do = round_to_dtype(normal(cfg, 4, (B, H, S, D)), dtype)
    m = round_to_dtype(normal(cfg, 3, (B, H, S, S)), dtype) if with_mask else None
    return q, k, v, do, m


def _max_err(got, want):
    assert np.all(np.isfinite(got)), "non-finite output"
    return float(np.max(np.abs(got.astype(np.float64) - want)))


MODES = [("plain", False, False), ("causal", True, False), ("bias", False, True)]

# fp32: the reference's budgets at (B2, H2, S96), abs error vs the f64 oracle
# (tests/kernels/attention/generic.mojo:440,485,530,575,620,665)
F32_CASES = [(64, 5e-6), (256, 2e-5), (512, 5e-5), (8, 5e-6), (40, 5e-6), (128, 1e-5)]


@pytest.mark.parametrize("name,causal,with_mask", MODES)
@pytest.mark.parametrize("D,budget", F32_CASES)
def test_f32_error_budget(device, name, causal, with_mask, D, budget):
    B, H, S = 2, 2, 96
    q, k, v, do, m = _inputs(50, B, S, H, D, F32, with_mask)
    o, lse, dq, dk, dv = _fwd_bwd(device, q, k, v, do, m, causal)
    ro, rl = O.sdpa_fwd(q, k, v, m, causal)
    rdq, rdk, rdv = O.sdpa_bwd(q, k, v, do, m, causal)
    assert _max_err(o, ro) <= budget and _max_err(lse, rl) <= budget
    assert _max_err(dq, rdq) <= budget and _max_err(dk, rdk) <= budget and _max_err(dv, rdv) <= budget


@pytest.mark.parametrize("name,causal,with_mask", MODES)
@pytest.mark.parametrize("B,H,S,D,budget", [(1, 2, 300, 64, 5e-6), (2, 1, 100, 128, 1e-5), (1, 3, 64, 24, 5e-6),
                                            (1, 1, 257, 72, 1e-5), (2, 2, 130, 32, 5e-6), (1, 2, 150, 256, 2e-5),
                                            (1, 1, 97, 200, 2e-5), (1, 2, 70, 512, 4e-5), (1, 1, 131, 328, 4e-5)])
def test_f32_row_per_thread_and_wave_per_row_kernels(device, monkeypatch, name, causal, with_mask, B, H, S, D, budget):
    # fp32 tensors with at least 64 tokens take kernels that keep a row per thread (or per 2 to
    # 16 neighbouring threads, 32 elements of the head each) and stage the other side through LDS;
    # MOGRAD_HIP_ATTN_TILED=0 keeps a wave per row.  Both must meet the reference's fp32 budget
    # against the f64 oracle, at sequence lengths that leave ragged tiles and idle threads.
    q, k, v, do, m = _inputs(58, B, S, H, D, F32, with_mask)
    ro, rl = O.sdpa_fwd(q, k, v, m, causal)
    want = (ro, rl) + tuple(O.sdpa_bwd(q, k, v, do, m, causal))
    monkeypatch.setenv("MOGRAD_HIP_ATTN_F32_MFMA", "0")  # (the matrix-core form has its own test below)
    for mode in ("0", "1"):
        monkeypatch.setenv("MOGRAD_HIP_ATTN_TILED", mode)
        got = _fwd_bwd(device, q, k, v, do, m, causal)
        for g, w, what in zip(got, want, ("o", "lse", "dq", "dk", "dv")):
            assert _max_err(g, w) <= budget, f"{what} (tiled={mode}): {_max_err(g, w)}"


@pytest.mark.parametrize("name,causal,with_mask", MODES)
@pytest.mark.parametrize("B,H,S,D,budget", [(1, 2, 300, 64, 5e-6), (2, 2, 96, 64, 5e-6), (1, 3, 64, 24, 5e-6),
                                            (2, 2, 130, 32, 5e-6), (1, 1, 257, 40, 5e-6), (1, 2, 129, 7, 5e-6),
                                            (1, 1, 1000, 64, 1e-5), (1, 2, 128, 48, 5e-6), (2, 1, 100, 128, 1e-5),
                                            (1, 1, 257, 72, 1e-5), (1, 2, 130, 100, 1e-5), (1, 2, 96, 16, 5e-6)])
def test_f32_matrix_core_kernels(device, monkeypatch, name, causal, with_mask, B, H, S, D, budget):
    # fp32 tensors with heads of up to 128 columns and at least 64 tokens take fp32 MFMA kernels
    # (32 resident rows per wave, tiles of 32 streamed rows; kernels for 32, 64 and 128 columns); they must meet the reference's fp32
    # budget against the f64 oracle like the FMA forms (tests/kernels/attention/generic.mojo:440-665),
    # at lengths that leave ragged tiles and blocks, head dims that are not multiples of four
    # (element-wise loads and stores) and both layouts of O.
    q, k, v, do, m = _inputs(60, B, S, H, D, F32, with_mask)
    ro, rl = O.sdpa_fwd(q, k, v, m, causal)
    want = (ro, rl) + tuple(O.sdpa_bwd(q, k, v, do, m, causal))
    results = {}
    for mfma in ("1", "0"):
        monkeypatch.setenv("MOGRAD_HIP_ATTN_F32_MFMA", mfma)
        results[mfma] = _fwd_bwd(device, q, k, v, do, m, causal)
        for g, w, what in zip(results[mfma], want, ("o", "lse", "dq", "dk", "dv")):
            assert _max_err(g, w) <= budget, f"{what} (mfma={mfma}): {_max_err(g, w)}"
    # and it is deterministic
    monkeypatch.setenv("MOGRAD_HIP_ATTN_F32_MFMA", "1")
    again = _fwd_bwd(device, q, k, v, do, m, causal)
    for a_, b_ in zip(again, results["1"]):
        np.testing.assert_array_equal(a_, b_)


HALF_SHAPES = [(2, 2, 96, 64), (1, 3, 200, 64), (2, 1, 128, 128), (1, 2, 257, 32), (1, 1, 4, 8), (1, 2, 96, 256),
               (1, 2, 130, 72), (1, 1, 80, 512), (1, 2, 40, 192), (1, 2, 300, 256), (2, 1, 130, 200), (1, 1, 129, 136)]


@pytest.mark.parametrize("dtype,budget_fwd,budget_bwd", [(F16, 2e-3, 8e-3), (BF16, 1.6e-2, 6.4e-2)])
@pytest.mark.parametrize("name,causal,with_mask", MODES)
@pytest.mark.parametrize("B,H,S,D", HALF_SHAPES)
def test_half_error_budget(device, dtype, budget_fwd, budget_bwd, name, causal, with_mask, B, H, S, D):
    # fp16: the reference's budget for its tensor-core backward is 8e-3 abs at S96
    # (tests/kernels/attention/mma.mojo:424); bf16 has 3 fewer mantissa bits: x8.
    q, k, v, do, m = _inputs(51, B, S, H, D, dtype, with_mask)
    o, lse, dq, dk, dv = _fwd_bwd(device, q, k, v, do, m, causal, dtype=dtype)
    ro, rl = O.sdpa_fwd(q, k, v, m, causal)
    # The backward is checked against the oracle's gradients at the O the kernel saw (its
    # own forward output, rounded to the storage type) entering only through delta.
    rdq, rdk, rdv = O.sdpa_bwd(q, k, v, do, m, causal)
    grow = math.sqrt(S / 96.0)
    assert _max_err(o, ro) <= budget_fwd
    assert _max_err(lse, rl) <= 1e-3 * max(1.0, float(np.abs(rl).max()))
    for got, want, what in ((dq, rdq, "dq"), (dk, rdk, "dk"), (dv, rdv, "dv")):
        err = _max_err(got, want)
        assert err <= budget_bwd * grow, f"{what}: {err}"


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_long_ragged_sequence(device, causal, D):
    # Past 1024 tokens the head-dim-64 backward launches its dK/dV and dQ walks separately
    # (one launch below that); 1100 is not a multiple of any tile.  Head dims 128 and 256: the
    # unpipelined walks, at 256 with the head dimension of the gradients split over two workgroups.
    B, H, S = 1, 2, 1100
    q, k, v, do, _ = _inputs(56, B, S, H, D, BF16, False)
    o, lse, dq, dk, dv = _fwd_bwd(device, q, k, v, do, None, causal, dtype=BF16)
    ro, rl = O.sdpa_fwd(q, k, v, None, causal)
    assert _max_err(o, ro) <= 1.6e-2 and _max_err(lse, rl) <= 1e-3 * max(1.0, float(np.abs(rl).max()))
    for got, want, what in zip((dq, dk, dv), O.sdpa_bwd(q, k, v, do, None, causal), ("dq", "dk", "dv")):
        assert_attn_grad_close(got, want, what)


@pytest.mark.parametrize("causal", [True, False])
def test_bf16_gradients_rtol(device, causal):
    # Parity bar for bf16 attention gradients: rtol 2e-2, with an absolute floor for entries that
    # cancel to ~0 of 7.5e-3 of the largest entry of the same (batch, head), twice the worst
    # excess observed (helpers.ATTN_BF16_FLOOR).
    B, H, S, D = 2, 3, 256, 64
    q, k, v, do, _ = _inputs(4, B, S, H, D, BF16, False)
    _, _, dq, dk, dv = _fwd_bwd(device, q, k, v, do, None, causal, dtype=BF16)
    for got, want, what in zip((dq, dk, dv), O.sdpa_bwd(q, k, v, do, None, causal), ("dq", "dk", "dv")):
        assert_attn_grad_close(got, want, what)


@pytest.mark.parametrize("dtype,rtol", [(F16, RTOL_BF16_ATTN / 8), (BF16, RTOL_BF16_ATTN)])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,H,S", [(3, 2, 256), (2, 3, 200), (1, 2, 33), (2, 2, 1), (4, 3, 128), (1, 1, 225)])
def test_whole_head_in_lds_backward(device, monkeypatch, dtype, rtol, causal, B, H, S):
    # Sequences up to 256 tokens of 64-wide heads: the backward keeps a (batch, head)'s Q, K, V
    # and dO in LDS and computes delta itself, one workgroup per head
    # (MOGRAD_HIP_ATTN_RESIDENT=0: the streaming walks).  Both against the oracle, at every
    # length class: full tiles, a ragged last tile, fewer tiles than waves, a single token.
    D = 64
    q, k, v, do, _ = _inputs(57, B, S, H, D, dtype, False)
    want = O.sdpa_bwd(q, k, v, do, None, causal)
    results = {}
    for mode in ("0", "1"):
        monkeypatch.setenv("MOGRAD_HIP_ATTN_RESIDENT", mode)
        results[mode] = _fwd_bwd(device, q, k, v, do, None, causal, dtype=dtype)[2:]
        for got, ref, what in zip(results[mode], want, ("dq", "dk", "dv")):
            # (a single token has dq = dk = 0 exactly; the kernels leave the rounding of dP - delta)
            assert_attn_grad_close(got, ref, f"{what} ({mode})", rtol=rtol, floor=ATTN_BF16_FLOOR * rtol / RTOL_BF16_ATTN,
                                   min_top=1e-2)
    # the two paths round P and dS to 16 bits at the same points: they differ by summation order only
    for a, b_, ref, what in zip(results["1"], results["0"], want, ("dq", "dk", "dv")):
        assert np.max(np.abs(a - b_)) <= 0.5 * rtol * max(np.abs(ref).max(), 1e-2), what
    # and the resident path is deterministic
    again = _fwd_bwd(device, q, k, v, do, None, causal, dtype=dtype)[2:]
    for a, b_ in zip(again, results["1"]):
        np.testing.assert_array_equal(a, b_)


def test_closed_forms(device):
    B, S, H, D = 1, 128, 1, 8
    z = np.zeros((B, S, H, D), np.float32)
    v = normal(52, 0, (B, S, H, D))
    # Q = K = 0 causal, loss = sum(O): dV[j] = sum_{i>=j} 1/(i+1)   (tests/test_grad.mojo:1001-1023)
    for dtype, tol in ((F32, 1e-5), (F16, 2e-2), (BF16, 2e-2)):
        _, _, _, _, dv = _fwd_bwd(device, z, z, v, np.ones((B, H, S, D), np.float32), None, True, dtype=dtype)
        tail = np.array([sum(1.0 / (i + 1) for i in range(j, S)) for j in range(S)])
        np.testing.assert_allclose(dv[0, :, 0, :], np.repeat(tail[:, None], D, axis=1), rtol=tol, atol=tol)
    # causal row 0 is V[0]; uniform scores average V; T=2 known value  (tests/test_ops.mojo:903-946)
    q, k = normal(52, 1, (B, S, H, D)), normal(52, 2, (B, S, H, D))
    o, lse, *_ = _fwd_bwd(device, q, k, v, np.ones((B, H, S, D), np.float32), None, True)
    np.testing.assert_allclose(o[0, 0, 0], v[0, 0, 0], rtol=1e-6)
    o, lse, *_ = _fwd_bwd(device, z, z, v, np.ones((B, H, S, D), np.float32), None, False)
    np.testing.assert_allclose(o[0, 0], np.repeat(v[0, :, 0].mean(axis=0)[None], S, axis=0), atol=1e-6)
    np.testing.assert_allclose(lse, math.log(S), rtol=1e-6)


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("S", [96, 200])
def test_bias_at_any_alignment(device, D, S):
    # A bias whose rows are whole 8-byte groups is read a group at a time; one that starts at an
    # odd element of its allocation (or has S % 4 != 0, which the shapes above cover) is read element
    # by element into the same form.  The results must be the same bits.
    q, k, v, do, m = _inputs(59, 1, S, 2, D, BF16, True)
    aligned = _fwd_bwd(device, q, k, v, do, m, False, dtype=BF16)
    for offset in (1, 2, 3):
        shifted = _fwd_bwd(device, q, k, v, do, m, False, dtype=BF16, mask_offset=offset)
        for a, b_, what in zip(aligned, shifted, ("o", "lse", "dq", "dk", "dv")):
            np.testing.assert_array_equal(a, b_, err_msg=f"{what} at offset {offset}")


def test_bias_shift_invariance(device):
    # tests/kernels/attention/generic.mojo:322-366
    q, k, v, do, m = _inputs(53, 2, 40, 2, 64, F32, True)
    o1, l1, dq1, dk1, dv1 = _fwd_bwd(device, q, k, v, do, m)
    o2, l2, dq2, dk2, dv2 = _fwd_bwd(device, q, k, v, do, m + np.float32(3.0))
    assert _max_err(o1, o2.astype(np.float64)) < 1e-5 and _max_err(l2 - l1, np.full(l1.shape, 3.0)) < 1e-4
    assert _max_err(dq1, dq2.astype(np.float64)) < 1e-5 and _max_err(dk1, dk2.astype(np.float64)) < 1e-5


def test_large_logits_stay_finite(device):
    # softmax is max-subtracted: std-8 Q, K give logits in the hundreds
    B, S, H, D = 1, 64, 2, 64
    q, k = normal(54, 0, (B, S, H, D), std=8.0), normal(54, 1, (B, S, H, D), std=8.0)
    v, do = normal(54, 2, (B, S, H, D)), normal(54, 3, (B, H, S, D))
    o, lse, dq, dk, dv = _fwd_bwd(device, q, k, v, do)
    ro, rl = O.sdpa_fwd(q, k, v)
    assert _max_err(o, ro) < 1e-3 and _max_err(lse, rl) < 1e-3 * np.abs(rl).max()


def test_placeholder_mask_is_never_read(device):
    # has_bias False: the mask operand is a 1-element placeholder  (rewrites.mojo:94-103)
    q, k, v, do, _ = _inputs(55, 1, 33, 2, 64, F32, False)
    o, lse, dq, dk, dv = _fwd_bwd(device, q, k, v, do, None, True)
    rdq, rdk, rdv = O.sdpa_bwd(q, k, v, do, None, True)
    assert _max_err(dq, rdq) < 5e-6 and _max_err(dk, rdk) < 5e-6 and _max_err(dv, rdv) < 5e-6


def test_has_bias_defaults(device):
    # forward dispatch: has_bias defaults to True; backward: to `not is_causal`
    # (dispatch.mojo:393-395,453-455)
    q, k, v, do, m = _inputs(56, 1, 16, 1, 8, F32, True)
    node = Node("FLASH_ATTN", Layout(1, 1, 16, 8), F32,
                [Node.leaf(Layout(1, 16, 1, 8))] * 3 + [Node.leaf(Layout(1, 1, 16, 16))], {"scale": 0.5, "is_causal": False})
    bufs = [AnyBuffer.from_numpy(device, a) for a in (q, k, v, m)]
    o, lse = R.run(node, bufs, device)
    ro, _ = O.sdpa_fwd(q, k, v, m, False, 0.5)
    assert _max_err(o.to_numpy((1, 1, 16, 8)), ro) < 5e-6


def test_errors(device):
    buf = AnyBuffer.create(F32, device, 64)
    p = buf.data_ptr()
    lib, st = device.lib, device.stream
    with pytest.raises(MogradError, match=r"D=513 out of range \(1..512\)"):
        lib.mg_flash_attn_fwd(p, p, p, p, p, p, 1, 1, 1, 513, 1.0, 0, 0, F32, st)
    with pytest.raises(MogradError, match=r"D=0 out of range"):
        lib.mg_flash_attn_bwd(p, p, p, p, p, p, p, p, p, p, 1, 1, 1, 0, 1.0, 0, 0, F32, st)
    with pytest.raises(MogradError, match="causal attention with additive bias is not supported"):
        lib.mg_flash_attn_fwd(p, p, p, p, p, p, 1, 2, 1, 8, 1.0, 1, 1, F32, st)
    with pytest.raises(MogradError, match="unsupported dtype"):
        lib.mg_flash_attn_fwd(p, p, p, p, p, p, 1, 2, 1, 8, 1.0, 0, 0, R.int64, st)


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("name,causal,with_mask", MODES)
@pytest.mark.parametrize("B,H,S,D", [(2, 3, 200, 64), (1, 2, 130, 72), (2, 2, 96, 128), (1, 1, 4, 8), (1, 2, 77, 40)])
def test_bshd_output_forms_equal_the_standard_forms(device, dtype, name, causal, with_mask, B, H, S, D):
    # O written and dO/O read as (B,S,H,D): bit for bit the standard entry points with the
    # (B,H,S,D) <-> (B,S,H,D) copies done on the host.  LSE stays (B,H,S).
    lib, st = device.lib, device.stream
    q, k, v, do, m = _inputs(54, B, S, H, D, dtype, with_mask)
    bq, bk, bv, bdo = (AnyBuffer.from_numpy(device, a, dtype) for a in (q, k, v, do))
    bdo_bshd = AnyBuffer.from_numpy(device, np.ascontiguousarray(do.transpose(0, 2, 1, 3)), dtype)
    bm = AnyBuffer.from_numpy(device, m if with_mask else np.zeros(8, np.float32), dtype)
    n = B * S * H * D
    scale = 1.0 / math.sqrt(D)
    new = lambda count=n, dt=dtype: AnyBuffer.create(dt, device, count)
    o1, o2, lse1, lse2 = new(), new(), new(B * H * S, F32), new(B * H * S, F32)
    P = lambda b: b.data_ptr()
    lib.mg_flash_attn_fwd(P(bq), P(bk), P(bv), P(bm), P(o1), P(lse1), B, S, H, D, scale, int(causal), int(with_mask), dtype, st)
    lib.mg_flash_attn_fwd_bshd(P(bq), P(bk), P(bv), P(bm), P(o2), P(lse2), B, S, H, D, scale, int(causal), int(with_mask),
                               dtype, st)
    np.testing.assert_array_equal(o2.to_numpy((B, S, H, D)), o1.to_numpy((B, H, S, D)).transpose(0, 2, 1, 3))
    np.testing.assert_array_equal(lse2.to_numpy(), lse1.to_numpy())
    g1, g2 = [new() for _ in range(3)], [new() for _ in range(3)]
    lib.mg_flash_attn_bwd(P(bdo), P(o1), P(bq), P(bk), P(bv), P(bm), P(lse1), *(P(g) for g in g1), B, S, H, D, scale,
                          int(causal), int(with_mask), dtype, st)
    lib.mg_flash_attn_bwd_bshd(P(bdo_bshd), P(o2), P(bq), P(bk), P(bv), P(bm), P(lse2), *(P(g) for g in g2), B, S, H, D,
                               scale, int(causal), int(with_mask), dtype, st)
    for a, b, what in zip(g1, g2, ("dq", "dk", "dv")):
        np.testing.assert_array_equal(b.to_numpy(), a.to_numpy(), err_msg=what)


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("name,causal,with_mask", MODES)
@pytest.mark.parametrize("B,H,S,D", [(2, 3, 200, 64), (1, 2, 130, 72), (2, 2, 96, 128), (1, 1, 4, 8), (1, 2, 77, 40)])
def test_packed_qkv_forms_equal_the_separate_forms(device, dtype, name, causal, with_mask, B, H, S, D):
    # Q, K, V as slices of one (B,S,3,H,D) tensor and dQ, dK, dV written into one: bit for bit
    # the separate-tensor entry points (with O and dO in (B,S,H,D)).
    lib, st = device.lib, device.stream
    q, k, v, do, m = _inputs(55, B, S, H, D, dtype, with_mask)
    do_bshd = np.ascontiguousarray(do.transpose(0, 2, 1, 3))
    qkv = np.ascontiguousarray(np.stack([q, k, v], axis=2))  # (B, S, 3, H, D)
    bq, bk, bv, bdo, bqkv = (AnyBuffer.from_numpy(device, a, dtype) for a in (q, k, v, do_bshd, qkv))
    bm = AnyBuffer.from_numpy(device, m if with_mask else np.zeros(8, np.float32), dtype)
    n = B * S * H * D
    scale = 1.0 / math.sqrt(D)
    new = lambda count=n, dt=dtype: AnyBuffer.create(dt, device, count)
    P = lambda b: b.data_ptr()
    flags = (B, S, H, D, scale, int(causal), int(with_mask), dtype, st)
    o1, o2, lse1, lse2 = new(), new(), new(B * H * S, F32), new(B * H * S, F32)
    lib.mg_flash_attn_fwd_bshd(P(bq), P(bk), P(bv), P(bm), P(o1), P(lse1), *flags)
    lib.mg_flash_attn_fwd_packed(P(bqkv), P(bm), P(o2), P(lse2), *flags)
    np.testing.assert_array_equal(o2.to_numpy(), o1.to_numpy())
    np.testing.assert_array_equal(lse2.to_numpy(), lse1.to_numpy())
    g = [new() for _ in range(3)]
    dqkv = AnyBuffer.create(dtype, device, 3 * n, fill=7.0)
    lib.mg_flash_attn_bwd_bshd(P(bdo), P(o1), P(bq), P(bk), P(bv), P(bm), P(lse1), *(P(x) for x in g), *flags)
    lib.mg_flash_attn_bwd_packed(P(bdo), P(o2), P(bqkv), P(bm), P(lse2), P(dqkv), *flags)
    got = dqkv.to_numpy((B, S, 3, H, D))
    for i, what in enumerate(("dq", "dk", "dv")):
        np.testing.assert_array_equal(got[:, :, i], g[i].to_numpy((B, S, H, D)), err_msg=what)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,H,S,D", [(2, 3, 512, 64), (1, 2, 1100, 64), (1, 2, 300, 40)])
def test_backward_walk_variants_agree(device, monkeypatch, causal, B, H, S, D):
    # Head dims up to 64 without a bias have four forms of the backward: the software-pipelined
    # walks or the plain ones (MOGRAD_HIP_ATTN_DKDV_PIPE=0), each as one launch for both walks or
    # as two (MOGRAD_HIP_ATTN_FUSED_BWD_MAX_S=0).  One launch or two runs the same workgroup code:
    # no bit may differ.  Pipelined and plain walks round P and dS to 16 bits at the same points
    # but form S - lse differently (inside the product's accumulator, or after it): they agree to
    # a quarter of the tolerance, and each meets it against the float64 oracle.
    monkeypatch.setenv("MOGRAD_HIP_ATTN_RESIDENT", "0")
    q, k, v, do, _ = _inputs(59, B, S, H, D, BF16, False)
    want = O.sdpa_bwd(q, k, v, do, None, causal)
    results = {}
    for pipe in ("1", "0"):
        for fused_max in ("1024", "0"):
            monkeypatch.setenv("MOGRAD_HIP_ATTN_DKDV_PIPE", pipe)
            monkeypatch.setenv("MOGRAD_HIP_ATTN_FUSED_BWD_MAX_S", fused_max)
            results[pipe, fused_max] = _fwd_bwd(device, q, k, v, do, None, causal, dtype=BF16)[2:]
            for got, ref, what in zip(results[pipe, fused_max], want, ("dq", "dk", "dv")):
                assert_attn_grad_close(got, ref, f"{what} (pipe {pipe}, one launch up to {fused_max})")
    for pipe in ("1", "0"):
        for a, b_, what in zip(results[pipe, "1024"], results[pipe, "0"], ("dq", "dk", "dv")):
            np.testing.assert_array_equal(a, b_, err_msg=f"{what}: one launch against two (pipe {pipe})")
    for a, b_, ref, what in zip(results["1", "0"], results["0", "0"], want, ("dq", "dk", "dv")):
        top = np.abs(np.asarray(ref)).max(axis=(1, 3), keepdims=True)
        assert np.all(np.abs(a - b_) <= 0.25 * (RTOL_BF16_ATTN * np.abs(ref) + ATTN_BF16_FLOOR * top)), what


# The two attention configurations of the benchmark at their own shapes: causal
# (B8, H12, S1024, D64) runs dK/dV and dQ in one launch of 1536 workgroups; non-causal
# (B2, H12, S4096, D64) takes the separately launched walks with 128-query steps.
C4_SHAPES = [("causal", 1, 8, 12, 1024, 64, True, [(0, 0), (3, 7), (7, 11)]),
             ("full", 2, 2, 12, 4096, 64, False, [(0, 0), (1, 5), (1, 11)])]


@pytest.mark.parametrize("name,cfg,B,H,S,D,causal,heads", C4_SHAPES)
def test_benchmark_shapes_against_oracle(device, name, cfg, B, H, S, D, causal, heads):
    import os

    q, k, v = (round_to_dtype(normal(4, cfg * 10 + i, (B, S, H, D)), BF16) for i in range(3))
    do = round_to_dtype(normal(4, cfg * 10 + 3, (B, H, S, D)), BF16)
    o, lse, dq, dk, dv = _fwd_bwd(device, q, k, v, do, None, causal, dtype=BF16)
    for t in (o, lse, dq, dk, dv):
        assert np.all(np.isfinite(t))
    # float64 oracle on the first, a middle and the last (batch, head)
    for b, h in heads:
        sl = lambda t: t[b:b + 1, :, h:h + 1, :]  # noqa: E731
        ro, rl = O.sdpa_fwd(sl(q), sl(k), sl(v), None, causal)
        assert _max_err(o[b:b + 1, h:h + 1], ro) <= 1.6e-2, (b, h)
        assert _max_err(lse[b:b + 1, h:h + 1], rl) <= 1e-3 * max(1.0, float(np.abs(rl).max())), (b, h)
        want = O.sdpa_bwd(sl(q), sl(k), sl(v), do[b:b + 1, h:h + 1], None, causal)
        for got, ref, what in zip((dq, dk, dv), want, ("dq", "dk", "dv")):
            assert_attn_grad_close(sl(got), ref, f"{what} at (b{b}, h{h})")
    # every (batch, head): a second run gives the same bits, and the gradients are linear in
    # dO exactly for a power-of-two factor (delta, dP and dS double without rounding)
    o2, lse2, dq2, dk2, dv2 = _fwd_bwd(device, q, k, v, do, None, causal, dtype=BF16)
    for a, b_, what in zip((o, lse, dq, dk, dv), (o2, lse2, dq2, dk2, dv2), ("o", "lse", "dq", "dk", "dv")):
        np.testing.assert_array_equal(a, b_, err_msg=what)
    _, _, dq4, dk4, dv4 = _fwd_bwd(device, q, k, v, do * np.float32(4.0), None, causal, dtype=BF16)
    for a, b_, what in zip((dq, dk, dv), (dq4, dk4, dv4), ("dq", "dk", "dv")):
        np.testing.assert_array_equal(a * np.float32(4.0), b_, err_msg=f"{what} not linear in dO")
    # every (batch, head) against the second formulation in the library: the wave-per-row
    # kernels that do all arithmetic in fp32 (no matrix cores, no tiles)
    os.environ["MOGRAD_HIP_ATTN_GENERIC"] = "1"
    try:
        og, lg, dqg, dkg, dvg = _fwd_bwd(device, q, k, v, do, None, causal, dtype=BF16)
    finally:
        del os.environ["MOGRAD_HIP_ATTN_GENERIC"]
    assert _max_err(o, og.astype(np.float64)) <= 3.2e-2
    assert _max_err(lse, lg.astype(np.float64)) <= 2e-3 * max(1.0, float(np.abs(lg).max()))
    for got, ref, what in zip((dq, dk, dv), (dqg, dkg, dvg), ("dq", "dk", "dv")):
        ref = ref.astype(np.float64)
        # per (batch, head) floor: the largest entry of that head's gradient
        top = np.abs(ref).max(axis=(1, 3), keepdims=True)
        bound = 2 * RTOL_BF16_ATTN * (np.abs(ref) + top)
        worst = np.max(np.abs(got - ref) / bound)
        assert worst <= 1.0, f"{what} vs fp32-arithmetic kernels: worst {worst:.3g}"
