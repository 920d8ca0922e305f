"""Pins the CPU oracle (oracle/oracle_np.py, oracle/oracle_c.c) before anything is
checked against it: the reference's own golden vectors, closed forms, a library routine
(torch on CPU, float64) and brute-force loops.  No GPU."""
import ctypes as C
import math
import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch

from helpers import golden
from oracle import oracle_np as O

ROOT = Path(__file__).resolve().parent.parent
ORACLE_SO = ROOT / "oracle" / "liboracle_c.so"


# --------------------------------------------------------------------------- #
# LayerNorm — goldens from the reference's tests
# --------------------------------------------------------------------------- #


@pytest.mark.parametrize("g", golden("layer_norm_fwd"), ids=lambda g: g["cite"])
def test_ln_fwd_goldens(g):
    y = O.layer_norm_fwd(g["x"], g["gamma"], g["beta"], g["eps"])
    np.testing.assert_allclose(y, g["y"], atol=g["atol"])


@pytest.mark.parametrize("g", golden("layer_norm_bwd"), ids=lambda g: g["cite"])
def test_ln_bwd_goldens(g):
    got = dict(zip(("dx", "dgamma", "dbeta"), O.layer_norm_bwd(g["dy"], g["x"], g["gamma"], g["eps"])))
    checked = [k for k in got if k in g]
    assert checked
    for k in checked:
        np.testing.assert_allclose(got[k], g[k], atol=g["atol"], err_msg=k)


def test_ln_bwd_matches_torch_autograd_and_invariants():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(7, 33))
    g = rng.uniform(0.5, 1.5, size=33)
    b = rng.normal(size=33)
    dy = rng.normal(size=(7, 33))
    xt = torch.tensor(x, requires_grad=True)
    gt = torch.tensor(g, requires_grad=True)
    bt = torch.tensor(b, requires_grad=True)
    y = torch.nn.functional.layer_norm(xt, (33,), gt, bt, eps=1e-5)
    y.backward(torch.tensor(dy))
    np.testing.assert_allclose(O.layer_norm_fwd(x, g, b), y.detach().numpy(), rtol=1e-10, atol=1e-12)
    dx, dg, db = O.layer_norm_bwd(dy, x, g)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(dg, gt.grad.numpy(), rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-9, atol=1e-11)
    # gamma = 1: dx is orthogonal to 1 in every row, and to xhat as eps -> 0
    dx1, _, _ = O.layer_norm_bwd(dy, x, np.ones(33), eps=1e-14)
    mu, rstd = O.layer_norm_stats(x, 1e-14)
    np.testing.assert_allclose(dx1.sum(axis=1), 0, atol=1e-12)
    np.testing.assert_allclose((dx1 * (x - mu) * rstd).sum(axis=1), 0, atol=1e-10)


def test_ln_rank3_is_rows_of_last_dim():
    # rows = numel / cols (dispatch.mojo:336-340)
    rng = np.random.default_rng(1)
    x = rng.normal(size=(2, 3, 8))
    dy = rng.normal(size=(2, 3, 8))
    g = rng.normal(size=8)
    a = O.layer_norm_bwd(dy, x, g)
    b = O.layer_norm_bwd(dy.reshape(6, 8), x.reshape(6, 8), g)
    np.testing.assert_allclose(a[0].reshape(6, 8), b[0])
    np.testing.assert_allclose(a[1], b[1])


# --------------------------------------------------------------------------- #
# Cross-entropy — goldens
# --------------------------------------------------------------------------- #


@pytest.mark.parametrize("g", golden("cross_entropy"), ids=lambda g: g["cite"])
def test_ce_goldens(g):
    assert abs(O.cross_entropy(g["logits"], g["labels"]) - g["loss"]) < g["atol"]


@pytest.mark.parametrize("g", golden("cross_entropy_grad"), ids=lambda g: g["cite"])
def test_ce_grad_goldens(g):
    d = O.cross_entropy_grad(np.array(g["a"], dtype=np.float64).T, g["labels"], g["upstream"])
    np.testing.assert_allclose(d.T.reshape(-1), g["grad_a_flat"], atol=g["atol"])


def test_ce_grad_rows_sum_to_zero():
    # tests/test_grad.mojo:432-446
    d = O.cross_entropy_grad(np.ones((4, 10)), O.one_hot([0, 1, 2, 3], 10))
    np.testing.assert_allclose(d.sum(axis=1), 0, atol=1e-12)


def test_ce_matches_torch_and_id_forms():
    rng = np.random.default_rng(2)
    x = rng.normal(scale=2, size=(9, 17))
    ids = rng.integers(0, 17, size=9)
    soft = rng.uniform(size=(9, 17))
    soft /= soft.sum(axis=1, keepdims=True)
    xt = torch.tensor(x, requires_grad=True)
    loss = torch.nn.functional.cross_entropy(xt, torch.tensor(ids))
    loss.backward()
    assert abs(O.cross_entropy_ids(x, ids) - loss.item()) < 1e-12
    assert abs(O.cross_entropy(x, O.one_hot(ids, 17)) - loss.item()) < 1e-12
    np.testing.assert_allclose(O.cross_entropy_grad_ids(x, ids), xt.grad.numpy(), atol=1e-13)
    np.testing.assert_allclose(O.cross_entropy_grad(x, O.one_hot(ids, 17), 1.0), xt.grad.numpy(), atol=1e-13)
    xt2 = torch.tensor(x, requires_grad=True)
    loss2 = torch.nn.functional.cross_entropy(xt2, torch.tensor(soft))
    (loss2 * 0.7).backward()
    assert abs(O.cross_entropy(x, soft) - loss2.item()) < 1e-12
    np.testing.assert_allclose(O.cross_entropy_grad(x, soft, 0.7), xt2.grad.numpy(), atol=1e-13)


def test_ce_rank3_matches_reshape():
    # tests/test_ops.mojo:178-186, tests/test_grad.mojo:467-483
    x = (np.arange(24) * 0.1).reshape(2, 3, 4)
    y = O.one_hot([0, 2, 1, 3, 0, 1], 4).reshape(2, 3, 4)
    assert abs(O.cross_entropy(x, y) - O.cross_entropy(x.reshape(6, 4), y.reshape(6, 4))) < 1e-14
    np.testing.assert_allclose(O.cross_entropy_grad(x, y).reshape(6, 4),
                               O.cross_entropy_grad(x.reshape(6, 4), y.reshape(6, 4)))


# --------------------------------------------------------------------------- #
# Attention — closed forms, brute force, library
# --------------------------------------------------------------------------- #


def test_sdpa_closed_forms():
    rng = np.random.default_rng(3)
    B, S, H, D = 1, 128, 1, 8
    v = rng.normal(size=(B, S, H, D))
    z = np.zeros((B, S, H, D))
    # tests/test_grad.mojo:1001-1023: Q = K = 0 causal, loss = sum(O):
    # dV[j] = sum_{i >= j} 1/(i+1)
    _, _, dv = O.sdpa_bwd(z, z, v, np.ones((B, H, S, D)), causal=True)
    tail = np.array([sum(1.0 / (i + 1) for i in range(j, S)) for j in range(S)])
    np.testing.assert_allclose(dv[0, :, 0, :], np.repeat(tail[:, None], D, axis=1), rtol=1e-12)
    # tests/test_ops.mojo:903-919: causal row 0 attends only to itself
    q = rng.normal(size=(B, S, H, D))
    k = rng.normal(size=(B, S, H, D))
    o, lse = O.sdpa_fwd(q, k, v, causal=True)
    np.testing.assert_allclose(o[0, 0, 0], v[0, 0, 0], rtol=1e-12)
    # tests/test_ops.mojo:932-946: uniform scores average V
    o, lse = O.sdpa_fwd(z, z, v)
    np.testing.assert_allclose(o[0, 0], np.repeat(v[0, :, 0].mean(axis=0)[None], S, axis=0), rtol=1e-12)
    np.testing.assert_allclose(lse, math.log(S))


def test_sdpa_bias_shift_invariance():
    # tests/kernels/attention/generic.mojo:322-366: a constant added to the bias changes
    # LSE by that constant and nothing else
    rng = np.random.default_rng(4)
    B, S, H, D = 2, 9, 2, 4
    q, k, v = (rng.normal(size=(B, S, H, D)) for _ in range(3))
    m = rng.normal(size=(B, H, S, S))
    o1, l1 = O.sdpa_fwd(q, k, v, mask=m)
    o2, l2 = O.sdpa_fwd(q, k, v, mask=m + 3.0)
    np.testing.assert_allclose(o1, o2, atol=1e-12)
    np.testing.assert_allclose(l2 - l1, 3.0, atol=1e-12)


@pytest.mark.parametrize("causal,has_mask", [(False, False), (True, False), (False, True)])
def test_sdpa_vectorised_equals_loops(causal, has_mask):
    rng = np.random.default_rng(5)
    B, S, H, D = 2, 7, 3, 5
    q, k, v = (rng.normal(size=(B, S, H, D)) for _ in range(3))
    do = rng.normal(size=(B, H, S, D))
    m = rng.normal(size=(B, H, S, S)) if has_mask else None
    scale = 0.37
    o, lse = O.sdpa_fwd(q, k, v, m, causal, scale)
    dq, dk, dv = O.sdpa_bwd(q, k, v, do, m, causal, scale)
    mflat = m.reshape(-1).tolist() if has_mask else []
    ol, ll = O.sdpa_fwd_loops(q.reshape(-1).tolist(), k.reshape(-1).tolist(), v.reshape(-1).tolist(), mflat, has_mask,
                              causal, B, S, H, D, scale)
    dql, dkl, dvl = O.sdpa_bwd_loops(q.reshape(-1).tolist(), k.reshape(-1).tolist(), v.reshape(-1).tolist(),
                                     do.reshape(-1).tolist(), mflat, has_mask, causal, B, S, H, D, scale)
    np.testing.assert_allclose(o.reshape(-1), ol, atol=1e-13)
    np.testing.assert_allclose(lse.reshape(-1), ll, atol=1e-13)
    np.testing.assert_allclose(dq.reshape(-1), dql, atol=1e-13)
    np.testing.assert_allclose(dk.reshape(-1), dkl, atol=1e-13)
    np.testing.assert_allclose(dv.reshape(-1), dvl, atol=1e-13)


@pytest.mark.parametrize("causal,has_mask", [(False, False), (True, False), (False, True)])
def test_sdpa_matches_torch_autograd(causal, has_mask):
    rng = np.random.default_rng(6)
    B, S, H, D = 2, 10, 2, 8
    q, k, v = (rng.normal(size=(B, S, H, D)) for _ in range(3))
    do = rng.normal(size=(B, H, S, D))
    m = rng.normal(size=(B, H, S, S)) if has_mask else None
    qt, kt, vt = (torch.tensor(a, requires_grad=True) for a in (q, k, v))
    out = torch.nn.functional.scaled_dot_product_attention(
        qt.transpose(1, 2), kt.transpose(1, 2), vt.transpose(1, 2),
        attn_mask=torch.tensor(m) if has_mask else None, is_causal=causal)
    out.backward(torch.tensor(do))
    o, _ = O.sdpa_fwd(q, k, v, m, causal)
    dq, dk, dv = O.sdpa_bwd(q, k, v, do, m, causal)
    np.testing.assert_allclose(o, out.detach().numpy(), atol=1e-12)
    np.testing.assert_allclose(dq, qt.grad.numpy(), atol=1e-12)
    np.testing.assert_allclose(dk, kt.grad.numpy(), atol=1e-12)
    np.testing.assert_allclose(dv, vt.grad.numpy(), atol=1e-12)


# --------------------------------------------------------------------------- #
# Linear gradients, relu_grad, pool classes
# --------------------------------------------------------------------------- #


def test_linear_grads_match_autograd():
    rng = np.random.default_rng(7)
    M, N, K = 5, 4, 6
    x, w, b = rng.normal(size=(M, K)), rng.normal(size=(N, K)), rng.normal(size=N)
    dy = rng.normal(size=(M, N))
    xt, wt, bt = (torch.tensor(a, requires_grad=True) for a in (x, w, b))
    y = torch.nn.functional.linear(xt, wt, bt)
    y.backward(torch.tensor(dy))
    np.testing.assert_allclose(O.matmul_bias_bt(x, w, b), y.detach().numpy(), atol=1e-13)
    np.testing.assert_allclose(O.linear_grad_x(dy, w), xt.grad.numpy(), atol=1e-13)
    np.testing.assert_allclose(O.linear_grad_w(dy, x), wt.grad.numpy(), atol=1e-13)
    np.testing.assert_allclose(O.linear_grad_b(dy), bt.grad.numpy(), atol=1e-13)
    out = np.maximum(y.detach().numpy(), 0)
    np.testing.assert_array_equal(O.relu_grad(out, dy), np.where(out > 0, dy, 0))


def test_round_class():
    # tests/test_memory.mojo:18-30 and mograd/memory.mojo:59-72
    for g in golden("pool_round_class"):
        assert O.round_class(g["nbytes"]) == g["class_bytes"], g
    assert O.round_class(512) == 512 and O.round_class(513) == 576
    assert O.round_class(4096) == 4096 and O.round_class(990) == 1024
    for n in [600, 5000, 123457, 1 << 20, (1 << 20) + 1, 3 << 28]:
        c = O.round_class(n)
        assert c >= n and (c - n) * 8 <= c and c % 64 == 0


# --------------------------------------------------------------------------- #
# The C restatement (fp32, OpenMP) against the float64 numpy oracle
# --------------------------------------------------------------------------- #


@pytest.fixture(scope="module")
def orc():
    if not ORACLE_SO.exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    lib = C.CDLL(str(ORACLE_SO))
    lib.orc_cross_entropy_f32.restype = C.c_float
    lib.orc_cross_entropy_ids_f32.restype = C.c_float
    lib.orc_round_class.restype = C.c_int64
    lib.orc_round_class.argtypes = [C.c_int64]
    return lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _l(v):
    return C.c_int64(v)


def test_c_oracle_layer_norm(orc):
    rng = np.random.default_rng(8)
    rows, cols = 37, 130
    x = rng.normal(size=(rows, cols)).astype(np.float32)
    dy = rng.normal(size=(rows, cols)).astype(np.float32)
    g = rng.uniform(0.5, 1.5, size=cols).astype(np.float32)
    b = rng.normal(size=cols).astype(np.float32)
    y = np.empty_like(x)
    orc.orc_layer_norm_fwd_f32(_p(x), _p(g), _p(b), _p(y), _l(rows), _l(cols), C.c_float(1e-5))
    np.testing.assert_allclose(y, O.layer_norm_fwd(x, g, b), rtol=1e-4, atol=1e-5)
    dx = np.empty_like(x)
    dg = np.empty_like(g)
    db = np.empty_like(g)
    orc.orc_layer_norm_bwd_f32(_p(dy), _p(x), _p(g), _p(dx), _p(dg), _p(db), _l(rows), _l(cols), C.c_float(1e-5), _l(8))
    rdx, rdg, rdb = O.layer_norm_bwd(dy, x, g)
    np.testing.assert_allclose(dx, rdx, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dg, rdg, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(db, rdb, rtol=1e-4, atol=1e-4)


def test_c_oracle_cross_entropy(orc):
    rng = np.random.default_rng(9)
    N, Cc = 19, 77
    x = rng.normal(scale=2, size=(N, Cc)).astype(np.float32)
    ids = rng.integers(0, Cc, size=N).astype(np.int32)
    y = O.one_hot(ids, Cc).astype(np.float32)
    up = np.array([0.5], dtype=np.float32)
    assert abs(orc.orc_cross_entropy_f32(_p(x), _p(y), _l(N), _l(Cc)) - O.cross_entropy(x, y)) < 1e-5
    assert abs(orc.orc_cross_entropy_ids_f32(_p(x), _p(ids), _l(N), _l(Cc)) - O.cross_entropy(x, y)) < 1e-5
    d = np.empty_like(x)
    orc.orc_cross_entropy_grad_f32(_p(x), _p(y), _p(up), _p(d), _l(N), _l(Cc))
    np.testing.assert_allclose(d, O.cross_entropy_grad(x, y, 0.5), rtol=1e-4, atol=1e-7)
    orc.orc_cross_entropy_grad_ids_f32(_p(x), _p(ids), _p(up), _p(d), _l(N), _l(Cc))
    np.testing.assert_allclose(d, O.cross_entropy_grad(x, y, 0.5), rtol=1e-4, atol=1e-7)


def test_c_oracle_linear(orc):
    rng = np.random.default_rng(10)
    M, N, K = 13, 11, 17
    x = rng.normal(size=(M, K)).astype(np.float32)
    w = rng.normal(size=(N, K)).astype(np.float32)
    b = rng.normal(size=N).astype(np.float32)
    dy = rng.normal(size=(M, N)).astype(np.float32)
    y = np.empty((M, N), np.float32)
    orc.orc_matmul_bias_bt_f32(_p(x), _p(w), _p(b), _p(y), _l(M), _l(N), _l(K))
    np.testing.assert_allclose(y, O.matmul_bias_bt(x, w, b), rtol=1e-4, atol=1e-5)
    dx = np.empty((M, K), np.float32)
    dw = np.empty((N, K), np.float32)
    db = np.empty(N, np.float32)
    orc.orc_linear_grad_x_f32(_p(dy), _p(w), _p(dx), _l(M), _l(N), _l(K))
    orc.orc_linear_grad_w_f32(_p(dy), _p(x), _p(dw), _l(M), _l(N), _l(K))
    orc.orc_linear_grad_b_f32(_p(dy), _p(db), _l(M), _l(N))
    np.testing.assert_allclose(dx, O.linear_grad_x(dy, w), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dw, O.linear_grad_w(dy, x), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(db, O.linear_grad_b(dy), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("causal,has_mask", [(False, False), (True, False), (False, True)])
def test_c_oracle_attention(orc, causal, has_mask):
    rng = np.random.default_rng(11)
    B, S, H, D = 2, 21, 2, 8
    q, k, v = (rng.normal(size=(B, S, H, D)).astype(np.float32) for _ in range(3))
    do = rng.normal(size=(B, H, S, D)).astype(np.float32)
    m = rng.normal(size=(B, H, S, S)).astype(np.float32)
    scale = 1 / math.sqrt(D)
    o = np.empty((B, H, S, D), np.float32)
    lse = np.empty((B, H, S), np.float32)
    orc.orc_sdpa_fwd_f32(_p(q), _p(k), _p(v), _p(m), int(has_mask), int(causal), _p(o), _p(lse), _l(B), _l(S), _l(H),
                         _l(D), C.c_float(scale), _l(B * H))
    ro, rl = O.sdpa_fwd(q, k, v, m if has_mask else None, causal, scale)
    np.testing.assert_allclose(o, ro, atol=5e-6)
    np.testing.assert_allclose(lse, rl, atol=5e-6)
    dq, dk, dv = (np.empty_like(q) for _ in range(3))
    orc.orc_sdpa_bwd_f32(_p(q), _p(k), _p(v), _p(do), _p(m), int(has_mask), int(causal), _p(dq), _p(dk), _p(dv),
                         _l(B), _l(S), _l(H), _l(D), C.c_float(scale), _l(B * H))
    rdq, rdk, rdv = O.sdpa_bwd(q, k, v, do, m if has_mask else None, causal, scale)
    # the reference's own budget for an fp32 backward at this size: 5e-6 abs
    # (tests/kernels/attention/generic.mojo:440)
    np.testing.assert_allclose(dq, rdq, atol=5e-6)
    np.testing.assert_allclose(dk, rdk, atol=5e-6)
    np.testing.assert_allclose(dv, rdv, atol=5e-6)


# --------------------------------------------------------------------------- #
# Embedding lookup / scatter-add and the whole transformer step
# --------------------------------------------------------------------------- #


def test_gather_scatter_add_pins():
    rng = np.random.default_rng(21)
    V, d, n = 7, 5, 40
    w = rng.normal(size=(V, d))
    y = rng.normal(size=(n, d))
    idx = rng.integers(0, V, size=n)
    idx[:3] = 2  # repeats are the point
    g = O.gather(w, idx)
    for i in range(n):
        np.testing.assert_array_equal(g[i], w[idx[i]])
    sa = O.scatter_add(idx, y, V)
    # adjoint identity: <gather(W, i), Y> = <W, scatter_add(i, Y)>
    assert abs((g * y).sum() - (w * sa).sum()) < 1e-10
    # library routine
    ref = torch.zeros(V, d, dtype=torch.float64).index_add_(0, torch.from_numpy(idx), torch.from_numpy(y)).numpy()
    np.testing.assert_allclose(sa, ref, atol=1e-12)
    # a row nobody indexes stays zero
    idx2 = np.where(idx == 4, 3, idx)
    assert not O.scatter_add(idx2, y, V)[4].any()
    # (B, T) index arrays flatten row-major
    np.testing.assert_array_equal(O.gather(w, idx.reshape(4, 10)).reshape(n, d), g)


def tiny_params(rng, V, d, ff, layers):
    def lin(o, i):
        b = math.sqrt(6.0 / i)
        return rng.uniform(-b, b, size=(o, i))

    blocks = []
    for _ in range(layers):
        blocks.append({
            "ln1_g": rng.uniform(0.5, 1.5, d), "ln1_b": rng.normal(0, 0.1, d),
            "wq": lin(d, d), "wk": lin(d, d), "wv": lin(d, d), "wo": lin(d, d),
            "ln2_g": rng.uniform(0.5, 1.5, d), "ln2_b": rng.normal(0, 0.1, d),
            "w1": lin(ff, d), "b1": rng.uniform(-0.1, 0.1, ff), "w2": lin(d, ff),
        })
    return {"embed": rng.normal(size=(V, d)), "lm_head": lin(V, d), "blocks": blocks}


def torch_tiny_transformer(params, ids, labels, n_heads, eps=1e-5):
    """The same model written with torch modules' functional forms and autograd (f64)."""
    F = torch.nn.functional
    leaf = lambda a: torch.tensor(np.asarray(a), dtype=torch.float64, requires_grad=True)
    tp = {"embed": leaf(params["embed"]), "lm_head": leaf(params["lm_head"]),
          "blocks": [{k: leaf(v) for k, v in b.items()} for b in params["blocks"]]}
    B, T = ids.shape
    d = tp["embed"].shape[1]
    h = F.embedding(torch.from_numpy(ids), tp["embed"])
    for b in tp["blocks"]:
        x1 = F.layer_norm(h, (d,), b["ln1_g"], b["ln1_b"], eps)
        q, k, v = (F.linear(x1, b[w]).reshape(B, T, n_heads, d // n_heads).transpose(1, 2) for w in ("wq", "wk", "wv"))
        ctx = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(B, T, d)
        h = h + F.linear(ctx, b["wo"])
        x2 = F.layer_norm(h, (d,), b["ln2_g"], b["ln2_b"], eps)
        h = h + F.linear(F.relu(F.linear(x2, b["w1"], b["b1"])), b["w2"])
    logits = F.linear(h, tp["lm_head"])
    loss = F.cross_entropy(logits.reshape(B * T, -1), torch.from_numpy(labels).reshape(-1))
    loss.backward()
    grads = {"embed": tp["embed"].grad.numpy(), "lm_head": tp["lm_head"].grad.numpy(),
             "blocks": [{k: v.grad.numpy() for k, v in b.items()} for b in tp["blocks"]]}
    return loss.item(), grads


def test_tiny_transformer_step_vs_torch_autograd():
    rng = np.random.default_rng(33)
    V, d, ff, layers, heads, B, T = 11, 16, 40, 2, 2, 3, 9
    params = tiny_params(rng, V, d, ff, layers)
    ids = rng.integers(0, V, size=(B, T))
    labels = rng.integers(0, V, size=(B, T))
    loss, grads = O.tiny_transformer_step(params, ids, labels, heads)
    tl, tg = torch_tiny_transformer(params, ids, labels, heads)
    assert abs(loss - tl) < 1e-12
    np.testing.assert_allclose(grads["embed"], tg["embed"], atol=1e-12)
    np.testing.assert_allclose(grads["lm_head"], tg["lm_head"], atol=1e-12)
    for g, t in zip(grads["blocks"], tg["blocks"]):
        assert set(g) == set(t)
        for name in g:
            np.testing.assert_allclose(g[name], t[name], atol=1e-12, err_msg=name)


def test_tiny_transformer_step_finite_difference():
    rng = np.random.default_rng(34)
    V, d, ff, layers, heads, B, T = 5, 8, 12, 1, 2, 2, 4
    params = tiny_params(rng, V, d, ff, layers)
    ids = rng.integers(0, V, size=(B, T))
    labels = rng.integers(0, V, size=(B, T))
    _, grads = O.tiny_transformer_step(params, ids, labels, heads)
    h = 1e-6
    for name, pos in [("wq", (1, 2)), ("w2", (3, 5)), ("b1", (4,)), ("ln1_g", (2,)), ("ln2_b", (6,))]:
        base = params["blocks"][0][name]
        up = base.copy(); up[pos] += h
        dn = base.copy(); dn[pos] -= h
        lu, _ = O.tiny_transformer_step({**params, "blocks": [{**params["blocks"][0], name: up}]}, ids, labels, heads)
        ld, _ = O.tiny_transformer_step({**params, "blocks": [{**params["blocks"][0], name: dn}]}, ids, labels, heads)
        assert abs((lu - ld) / (2 * h) - grads["blocks"][0][name][pos]) < 1e-7, name


@pytest.mark.parametrize("decoupled,wd", [(False, 0.0), (False, 0.1), (True, 0.1), (True, 0.0)])
def test_adam_and_sgd_vs_torch_optim(decoupled, wd):
    rng = np.random.default_rng(50)
    w0 = rng.normal(size=37)
    grads = [rng.normal(size=37) * s for s in (1.0, 0.1, 3.0, 1e-3)]
    lr, b1, b2, eps = 3e-3, 0.9, 0.999, 1e-8
    p = torch.tensor(w0, dtype=torch.float64, requires_grad=True)
    opt = (torch.optim.AdamW if decoupled else torch.optim.Adam)([p], lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd)
    w, m, v = w0.copy(), np.zeros(37), np.zeros(37)
    for t, g in enumerate(grads, start=1):
        p.grad = torch.tensor(g, dtype=torch.float64)
        opt.step()
        w, m, v = O.adam_step(w, g, m, v, lr, b1, b2, eps, wd, t, decoupled)
        np.testing.assert_allclose(w, p.detach().numpy(), rtol=1e-12, atol=1e-14)
    p = torch.tensor(w0, dtype=torch.float64, requires_grad=True)
    opt = torch.optim.SGD([p], lr=0.05)
    p.grad = torch.tensor(grads[0], dtype=torch.float64)
    opt.step()
    np.testing.assert_allclose(O.sgd_step(w0, grads[0], 0.05), p.detach().numpy(), rtol=1e-15)


def test_softmax_and_argmax_pins():
    rng = np.random.default_rng(60)
    x = rng.normal(size=(5, 3, 17)) * 4
    up = rng.normal(size=(5, 3, 17))
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    ty = torch.softmax(tx, dim=-1)
    ty.backward(torch.tensor(up))
    y = O.softmax(x)
    np.testing.assert_allclose(y, ty.detach().numpy(), atol=1e-15)
    np.testing.assert_allclose(y.sum(-1), 1.0, atol=1e-14)
    g = O.softmax_grad(y, up)
    np.testing.assert_allclose(g, tx.grad.numpy(), atol=1e-14)
    np.testing.assert_allclose(g.sum(-1), 0.0, atol=1e-14)  # the softmax Jacobian annihilates constants
    # argmax: first occurrence, like numpy on NaN-free data, along any axis
    a = rng.integers(0, 4, size=(6, 7, 5)).astype(np.float64)  # many ties
    for axis in (0, 1, 2, -1):
        np.testing.assert_array_equal(O.argmax_axis(a, axis), np.argmax(a, axis=axis))
    # hand cases for the reference's loop: NaN never wins, all -inf or all NaN gives 0
    assert O.argmax_axis([[np.nan, 1.0, 3.0, 3.0]], -1)[0] == 2
    assert O.argmax_axis([[np.nan, np.nan]], -1)[0] == 0
    assert O.argmax_axis([[-np.inf, -np.inf]], -1)[0] == 0
    assert O.argmax_axis([[2.0, np.nan, 5.0, np.nan]], -1)[0] == 2


def test_c_oracle_round_class(orc):
    for n in [1, 512, 513, 990, 1000, 1024, 1025, 4096, 5000, 123457, (1 << 20) + 1]:
        assert orc.orc_round_class(n) == O.round_class(n)
