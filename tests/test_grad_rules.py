"""Gradient rules of the host mirror: the rules of mograd/grad.mojo that lie on the backward
hot path, and the ones the reference lacks (a fused Linear backward for MATMUL_BT /
MATMUL_BIAS_BT, LayerNorm as a multi-output node whose statistics feed the backward,
cross-entropy on class ids), driven the way Tensor.gradient drives them: Grad.compute over
the graph (mograd/grad.mojo:22-91), then the scheduler's evaluation of the gradient nodes
(mograd/scheduler.mojo:40-80)."""
import numpy as np
import pytest

from helpers import ATOL_F32, RTOL_F32, assert_close, assert_sum_close, integers, normal, uniform
from oracle import oracle_np as O

from mograd_amd import BF16, F32, I32, I64, AnyBuffer, Layout, Node
from mograd_amd import runtime as R
from mograd_amd.runtime import round_to_dtype


# ---- graph structure: no GPU ------------------------------------------------------------------


def test_linear_rule_emits_one_multi_output_node():
    x, w, b = Node.leaf(Layout(4, 8)), Node.leaf(Layout(6, 8)), Node.leaf(Layout(6))
    y = Node("MATMUL_BIAS_BT", Layout(4, 6), F32, [x, w, b])
    dy = Node.leaf(Layout(4, 6))
    dx, dw, db = R.gradient(y, dy, [x, w, b])
    assert [g.op_type for g in (dx, dw, db)] == ["GETTUPLE"] * 3
    assert [g.attrs()["index"] for g in (dx, dw, db)] == [0, 1, 2]
    bwd = dx.src(0)
    assert bwd is dw.src(0) and bwd is db.src(0), "one LINEAR_GRAD node serves all three gradients"
    assert bwd.op_type == "LINEAR_GRAD" and bwd.srcs == [dy, x, w] and bwd.attrs()["has_bias"] is True
    assert (dx.layout().shape(), dw.layout().shape(), db.layout().shape()) == ((4, 8), (6, 8), (6,))
    # without a bias: two gradients
    y2 = Node("MATMUL_BT", Layout(4, 6), F32, [x, w])
    g = R.gradient(y2, dy, [x, w])
    assert g[0].src(0).attrs()["has_bias"] is False and len(R.GRAD_RULES["MATMUL_BT"](y2, dy)) == 2


def test_layer_norm_stats_rule_feeds_the_statistics_back():
    x, g, b = Node.leaf(Layout(3, 5, 16)), Node.leaf(Layout(16)), Node.leaf(Layout(16))
    ln = Node("LAYER_NORM_STATS", Layout(3, 5, 16), F32, [x, g, b], {"eps": 1e-5})
    y = Node("GETTUPLE", Layout(3, 5, 16), F32, [ln], {"index": 0})
    dy = Node.leaf(Layout(3, 5, 16))
    dx, dg, db = R.gradient(y, dy, [x, g, b])
    bwd = dx.src(0)
    assert bwd.op_type == "LAYER_NORM_STATS_GRAD" and bwd is dg.src(0) and bwd is db.src(0)
    up, bx, bg, mean, rstd = bwd.srcs
    assert up is dy and bx is x and bg is g
    assert mean.op_type == rstd.op_type == "GETTUPLE" and mean.src(0) is ln and rstd.src(0) is ln
    assert (mean.attrs()["index"], rstd.attrs()["index"]) == (1, 2)
    assert mean.layout().shape() == (15,) and mean.dtype() == F32  # rows = numel / cols


def test_reference_rules_on_the_path():
    # layer_norm_grad (mograd/grad.mojo:296-306) and cross_entropy_grad (:224-230)
    x, g, b = Node.leaf(Layout(4, 8)), Node.leaf(Layout(8)), Node.leaf(Layout(8))
    ln = Node("LAYER_NORM", Layout(4, 8), F32, [x, g, b], {"eps": 1e-5, "axis": -1})
    dx, dg, db = R.gradient(ln, Node.leaf(Layout(4, 8)), [x, g, b])
    assert dx.src(0).op_type == "LAYER_NORM_GRAD" and dx.src(0).attrs()["eps"] == 1e-5
    labels = Node.leaf(Layout(4, 8))
    ce = Node("CROSS_ENTROPY", Layout(1), F32, [ln, labels])
    one = Node.leaf(Layout(1))
    dlogits, dlabels = R.GRAD_RULES["CROSS_ENTROPY"](ce, one)
    assert dlabels is None and dlogits.op_type == "CROSS_ENTROPY_GRAD" and dlogits.srcs == [ln, labels, one]
    # flash_attn_grad (:309-344): O and LSE from the forward's outputs, LSE (B,H,S) f32, no mask gradient
    q = Node.leaf(Layout(2, 16, 3, 8))
    fa = Node("FLASH_ATTN", Layout(2, 3, 16, 8), F32, [q, q, q, Node.leaf(Layout(1))], {"scale": 0.5, "is_causal": True})
    grads = R.GRAD_RULES["FLASH_ATTN"](fa, Node.leaf(Layout(2, 3, 16, 8)))
    assert grads[3] is None and grads[0].src(0).op_type == "FLASH_ATTN_GRAD"
    lse = grads[0].src(0).src(6)
    assert lse.layout().shape() == (2, 3, 16) and lse.dtype() == F32 and lse.attrs()["index"] == 1
    # two paths into one node accumulate with ADD (Grad.accum, :93-95)
    y = Node("MATMUL_BT", Layout(4, 4), F32, [x, x])  # both operands are x
    gx, = R.gradient(y, Node.leaf(Layout(4, 4)), [x])
    assert gx.op_type == "ADD"
    with pytest.raises(R.MogradError, match="no gradient rule for op: CONV2D"):
        R.gradient(Node("CONV2D", Layout(4, 8), F32, [x]), Node.leaf(Layout(4, 8)), [x])


# ---- through the GPU -------------------------------------------------------------------------------


def _leaf(device, a, dtype=F32):
    from mograd_amd import AnyBuffer

    return Node.leaf(Layout(*a.shape), dtype, AnyBuffer.from_numpy(device, a, dtype))


def test_sum_and_expand_rules_are_each_others_gradient():
    # sum_grad (mograd/grad.mojo:156-177): the upstream as an EXPAND view with stride 0 along the
    # summed axis; expand_grad (:278-288): sums back over what EXPAND added or widened.
    x = Node.leaf(Layout(5, 7, 3))
    for axis, keep, up_shape, strides in ((1, False, (5, 3), (3, 0, 1)), (0, False, (7, 3), (0, 3, 1)),
                                          (2, True, (5, 7, 1), (7, 1, 0))):
        attrs = {"axis": axis, "keepdim": True} if keep else {"axis": axis}
        y = Node("SUM", Layout(*up_shape), F32, [x], attrs)
        (dx,) = R.gradient(y, Node.leaf(Layout(*up_shape)), [x])
        assert dx.op_type == "EXPAND" and dx.layout().shape() == (5, 7, 3) and dx.layout().stride() == strides
    full = Node("SUM", Layout(1), F32, [x])
    (dx,) = R.gradient(full, Node.leaf(Layout(1)), [x])
    assert dx.layout().stride() == (0, 0, 0)
    # EXPAND of a bias row over the rows of a matrix: its gradient is the column sum
    b = Node.leaf(Layout(6))
    e = Node("EXPAND", Layout(4, 6, strides=(0, 1)), F32, [b])
    (db,) = R.gradient(e, Node.leaf(Layout(4, 6)), [b])
    assert db.op_type == "SUM" and db.attrs()["axis"] == 0 and db.layout().shape() == (6,)
    # a widened size-1 axis keeps its dimension
    c = Node.leaf(Layout(4, 1))
    e2 = Node("EXPAND", Layout(4, 6, strides=(1, 0)), F32, [c])
    (dc,) = R.gradient(e2, Node.leaf(Layout(4, 6)), [c])
    assert dc.op_type == "SUM" and dc.attrs()["axis"] == 1 and dc.layout().shape() == (4, 1)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(64, 40, 256), (300, 136, 72)])
def test_sum_gradient_through_a_linear_layer(device, M, N, K):
    # s = sum over rows of (X W^T); ds/dX and ds/dW for an upstream g over the N columns: the
    # EXPAND view that sum_grad builds is materialised by the Linear backward's exec function.
    x, w, g = normal(66, 0, (M, K)), normal(66, 1, (N, K), std=0.1), normal(66, 2, (N,))
    nx, nw = (Node.leaf(Layout(*a.shape), F32, AnyBuffer.from_numpy(device, a)) for a in (x, w))
    h = Node("MATMUL_BT", Layout(M, N), F32, [nx, nw])
    s_ = Node("SUM", Layout(N), F32, [h], {"axis": 0})
    up = Node.leaf(Layout(N), F32, AnyBuffer.from_numpy(device, g))
    dx, dw = R.gradient(s_, up, [nx, nw])
    got_dx, got_dw = (b.to_numpy(shape) for b, shape in zip(R.evaluate_many([dx, dw], device), ((M, K), (N, K))))
    g64, x64, w64 = g.astype(np.float64), x.astype(np.float64), w.astype(np.float64)
    want_dx = np.broadcast_to(g64 @ w64, (M, K))
    want_dw = np.outer(g64, x64.sum(axis=0))
    assert_close(got_dx, want_dx, RTOL_F32, RTOL_F32 * np.abs(want_dx).max(), "dx")
    assert_close(got_dw, want_dw, RTOL_F32, RTOL_F32 * np.abs(want_dw).max(), "dw")
    assert_close(R.evaluate(s_, device).to_numpy(), (x64 @ w64.T).sum(axis=0), RTOL_F32, RTOL_F32 * M, "sum")


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(64, 10, 256), (200, 136, 260), (512, 384, 384)])
def test_linear_gradient_through_the_rule(device, M, N, K):
    x, w, b, dy = normal(80, 0, (M, K)), normal(80, 1, (N, K)), normal(80, 2, (N,)), normal(80, 3, (M, N))
    nx, nw, nb, ndy = (_leaf(device, a) for a in (x, w, b, dy))
    y = Node("MATMUL_BIAS_BT", Layout(M, N), F32, [nx, nw, nb])
    dx, dw, db = R.gradient(y, ndy, [nx, nw, nb])
    got = [R.evaluate(g, device).to_numpy(g.layout().shape()) for g in (dx, dw, db)]
    assert dx.src(0).bufs is not None and len(dx.src(0).bufs) == 3, "LINEAR_GRAD ran once, three outputs"
    assert_sum_close(got[0], O.linear_grad_x(dy, w), np.abs(dy) @ np.abs(w), what="dx")
    assert_sum_close(got[1], O.linear_grad_w(dy, x), np.abs(dy).T @ np.abs(x), what="dw")
    assert_sum_close(got[2], O.linear_grad_b(dy), np.abs(dy).sum(axis=0), what="db")
    # the node itself through the scheduler entry
    node = Node("LINEAR_GRAD", Layout(M, K), F32, [Node.leaf(Layout(M, N)), Node.leaf(Layout(M, K)), Node.leaf(Layout(N, K))],
                {"has_bias": False})
    out = R.run(node, [ndy.bufs[0], nx.bufs[0], nw.bufs[0]], device)
    assert len(out) == 2
    np.testing.assert_array_equal(out[1].to_numpy((N, K)), got[1])


@pytest.mark.gpu
def test_layer_norm_stats_gradient_equals_the_plain_rule(device):
    rows, cols = 300, 384
    x, dy = normal(81, 0, (rows, cols), mean=0.3), normal(81, 1, (rows, cols))
    g, b = uniform(81, 2, (cols,), 0.5, 1.5), normal(81, 3, (cols,), std=0.1)
    nx, ng, nb, ndy = (_leaf(device, a) for a in (x, g, b, dy))
    ln = Node("LAYER_NORM_STATS", Layout(rows, cols), F32, [nx, ng, nb], {"eps": 1e-5})
    y = Node("GETTUPLE", Layout(rows, cols), F32, [ln], {"index": 0})
    grads = R.gradient(y, ndy, [nx, ng, nb])
    got = [R.evaluate(t, device).to_numpy(t.layout().shape()) for t in grads]
    mean, rstd = (ln.bufs[i].to_numpy() for i in (1, 2))
    rmu, rrs = O.layer_norm_stats(x, 1e-5)
    assert_close(R.evaluate(y, device).to_numpy((rows, cols)), O.layer_norm_fwd(x, g, b), RTOL_F32, ATOL_F32, "y")
    assert_close(mean, rmu[:, 0], RTOL_F32, ATOL_F32, "mean")
    assert_close(rstd, rrs[:, 0], RTOL_F32, ATOL_F32, "rstd")
    rdx, rdg, rdb = O.layer_norm_bwd(dy, x, g)
    xhat = (x - rmu) * rrs
    assert_close(got[0], rdx, RTOL_F32, ATOL_F32, "dx")
    assert_sum_close(got[1], rdg, (np.abs(dy) * np.abs(xhat)).sum(axis=0), what="dgamma")
    assert_sum_close(got[2], rdb, np.abs(dy).sum(axis=0), what="dbeta")
    # the reference's single-output LAYER_NORM with its own rule gives the same gradients
    ln1 = Node("LAYER_NORM", Layout(rows, cols), F32, [nx, ng, nb], {"eps": 1e-5, "axis": -1})
    plain = [R.evaluate(t, device).to_numpy(t.layout().shape()) for t in R.gradient(ln1, ndy, [nx, ng, nb])]
    for a, c, what in zip(got, plain, ("dx", "dgamma", "dbeta")):
        assert_close(a, c, RTOL_F32, 10 * ATOL_F32, what + " stats vs plain")


@pytest.mark.gpu
@pytest.mark.parametrize("id_dtype,np_id", [(I32, np.int32), (I64, np.int64)])
def test_cross_entropy_ids_gradient(device, id_dtype, np_id):
    from mograd_amd import AnyBuffer

    n, c = 257, 1000
    logits = normal(82, 0, (n, c), std=2.0)
    ids = integers(82, 1, (n,), 0, c, np_id)
    nl = _leaf(device, logits)
    ni = Node.leaf(Layout(n), id_dtype, AnyBuffer.from_numpy(device, ids, id_dtype))
    loss = Node("CROSS_ENTROPY_IDS", Layout(1), F32, [nl, ni])
    one = _leaf(device, np.ones(1, np.float32))
    (dlogits,) = R.gradient(loss, one, [nl])
    assert dlogits.op_type == "CROSS_ENTROPY_IDS_GRAD"
    assert_close(R.evaluate(loss, device).item(), O.cross_entropy_ids(logits, ids), RTOL_F32, ATOL_F32, "loss")
    got = R.evaluate(dlogits, device).to_numpy((n, c))
    assert_close(got, O.cross_entropy_grad_ids(logits, ids), RTOL_F32, ATOL_F32 / n, "dlogits")
    neg = got < 0
    assert np.array_equal(neg.sum(axis=1), np.ones(n, np.int64)) and np.array_equal(np.argmax(neg, axis=1), ids)
    # equals the dense rule on one-hot rows
    dense = Node("CROSS_ENTROPY", Layout(1), F32, [nl, _leaf(device, O.one_hot(ids, c).astype(np.float32))])
    (dl2,) = R.gradient(dense, one, [nl])
    assert_close(R.evaluate(dl2, device).to_numpy((n, c)), got, RTOL_F32, ATOL_F32 / n, "dense vs ids")


@pytest.mark.gpu
def test_mlp_gradient_through_the_rules(device):
    # x -> Linear+bias -> ReLU -> LayerNorm (statistics kept) -> Linear+bias -> cross-entropy on ids:
    # every parameter gradient from gradient() + evaluate(), against the float64 oracle chain.
    from mograd_amd import AnyBuffer

    M, D0, D1, D2 = 64, 96, 128, 10
    x = normal(83, 0, (M, D0))
    w1, b1 = uniform(83, 1, (D1, D0), -0.25, 0.25), uniform(83, 2, (D1,), -0.25, 0.25)
    g, be = uniform(83, 3, (D1,), 0.5, 1.5), normal(83, 4, (D1,), std=0.1)
    w2, b2 = uniform(83, 5, (D2, D1), -0.2, 0.2), uniform(83, 6, (D2,), -0.2, 0.2)
    ids = integers(83, 7, (M,), 0, D2, np.int32)
    nx, nw1, nb1, ng, nbe, nw2, nb2 = (_leaf(device, a) for a in (x, w1, b1, g, be, w2, b2))
    ni = Node.leaf(Layout(M), I32, AnyBuffer.from_numpy(device, ids, I32))
    h_pre = Node("MATMUL_BIAS_BT", Layout(M, D1), F32, [nx, nw1, nb1])
    h = Node("RELU", Layout(M, D1), F32, [h_pre])
    ln = Node("LAYER_NORM_STATS", Layout(M, D1), F32, [h, ng, nbe], {"eps": 1e-5})
    y = Node("GETTUPLE", Layout(M, D1), F32, [ln], {"index": 0})
    logits = Node("MATMUL_BIAS_BT", Layout(M, D2), F32, [y, nw2, nb2])
    loss = Node("CROSS_ENTROPY_IDS", Layout(1), F32, [logits, ni])
    params = [nw1, nb1, ng, nbe, nw2, nb2]
    grads = R.gradient(loss, _leaf(device, np.ones(1, np.float32)), params)
    got = [R.evaluate(t, device).to_numpy(t.layout().shape()) for t in grads]
    # oracle
    r_hpre = O.matmul_bias_bt(x, w1, b1)
    r_h = np.maximum(r_hpre, 0)
    r_y = O.layer_norm_fwd(r_h, g, be)
    r_logits = O.matmul_bias_bt(r_y, w2, b2)
    assert_close(R.evaluate(loss, device).item(), O.cross_entropy_ids(r_logits, ids), RTOL_F32, ATOL_F32, "loss")
    r_dlogits = O.cross_entropy_grad_ids(r_logits, ids)
    r_dy = O.linear_grad_x(r_dlogits, w2)
    r_dh, r_dg, r_dbe = O.layer_norm_bwd(r_dy, r_h, g)
    r_dhpre = O.relu_grad(r_h, r_dh)
    want = [O.linear_grad_w(r_dhpre, x), O.linear_grad_b(r_dhpre), r_dg, r_dbe, O.linear_grad_w(r_dlogits, r_y),
            O.linear_grad_b(r_dlogits)]
    for a, c, what in zip(got, want, ("dw1", "db1", "dgamma", "dbeta", "dw2", "db2")):
        assert_close(a, c, RTOL_F32, ATOL_F32, what)


# --------------------------------------------------------------------------- #
# The transformer step through gradient() + Simplifier(GPU_REWRITES()) + evaluate_many()
# --------------------------------------------------------------------------- #


def _op_counts(roots):
    from mograd_amd.runtime import _toposort

    counts = {}
    for n in _toposort(Node("SINK", Layout(1), F32, list(roots)))[:-1]:
        counts[n.op_type] = counts.get(n.op_type, 0) + 1
    return counts


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [BF16, F32])
@pytest.mark.parametrize("V,d,ff,L,H,B,T", [(65, 128, 512, 2, 2, 4, 64), (65, 384, 1536, 1, 6, 16, 256)])
def test_transformer_step_through_the_rule_tables(device, dtype, V, d, ff, L, H, B, T):
    # The forward graph in plain ops (GATHER, LAYER_NORM_STATS, MATMUL_BT, ADD, RELU, MATMUL_BIAS_BT,
    # packed attention, cross-entropy on ids), differentiated by gradient() over GRAD_RULES, rewritten
    # into the fused nodes and evaluated: every parameter gradient and the loss must equal the
    # hand-sequenced TinyTransformer.step bit for bit, and the rewritten graph must consist of the
    # fused nodes that step calls (no separate ADD / RELU / RELU_GRAD left in a block).
    from helpers import integers
    from mograd_amd.tiny_transformer import TinyTransformer, init_params

    rng = np.random.Generator(np.random.PCG64(75_000 + d))
    params = init_params(rng, V, d, ff, L)
    for b in params["blocks"]:
        for g, be in (("ln1_g", "ln1_b"), ("ln2_g", "ln2_b")):
            b[g] = rng.uniform(0.5, 1.5, b[g].shape).astype(np.float32)
            b[be] = rng.normal(0, 0.1, b[be].shape).astype(np.float32)
    ids = AnyBuffer.from_numpy(device, integers(75, 1, (B, T), 0, V, np.int32))
    labels = AnyBuffer.from_numpy(device, integers(75, 2, (B, T), 0, V, np.int32))
    model = TinyTransformer(device, V, d, ff, L, H, compute_dtype=dtype, deferred=False)
    model.load_params(params)
    want_loss = model.step(ids, labels, B, T).item()
    want = model.gradients()
    for deferred_sums in (False, True):
        loss, grads, roots = model.step_via_rules(ids, labels, B, T, deferred_sums=deferred_sums)
        assert loss.item() == want_loss
        for name, buf in grads.items():
            parts = name.split(".")
            ref = want["blocks"][int(parts[1])] if parts[0] == "blocks" else want
            key = parts[-1]
            if key == "wq":  # the stacked (3d, d) projection: wq | wk | wv
                blk = want["blocks"][int(parts[1])]
                expect = np.concatenate([blk["wq"], blk["wk"], blk["wv"]], axis=0)
            else:
                expect = ref[key]
            np.testing.assert_array_equal(buf.to_numpy(expect.shape), expect, err_msg=f"{name} (deferred {deferred_sums})")
    counts = _op_counts(roots)
    assert counts.get("MATMUL_BT_ADD") == 2 * L and counts.get("MATMUL_BIAS_RELU_BT") == L
    # both LayerNorms of a block feed a Linear layer: their backward rides on that layer's
    assert counts.get("LINEAR_LAYER_NORM_GRAD") == 2 * L and counts.get("LINEAR_GRAD") == 2 * L + 1
    assert "LAYER_NORM_STATS_GRAD" not in counts and "LAYER_NORM_STATS_GRAD_ADD" not in counts
    from mograd_amd.runtime import _toposort
    assert all(nd.attrs().get("accumulate") for nd in _toposort(Node("SINK", Layout(1), F32, list(roots)))
               if nd.op_type == "LINEAR_LAYER_NORM_GRAD")
    for gone in ("ADD", "RELU", "RELU_GRAD"):
        assert gone not in counts, f"{gone} survived the rewrites: {counts}"


@pytest.mark.gpu
def test_rewrites_attention_copy_and_shared_input_accumulation(device):
    # (i) CONTIGUOUS(TRANSPOSE(FLASH_ATTN[0])) -> FLASH_ATTN{layout: bshd}, and its gradient node
    # follows; (ii) three projections of one input: their input gradients ADD(ADD(dx_q, dx_k), dx_v)
    # become accumulating LINEAR_GRAD nodes.  The rewritten graph must give the same bits as the
    # graph as written.
    from mograd_amd.rewrites import GPU_REWRITES, Simplifier
    from mograd_amd.runtime import evaluate_many

    B, S, H, D, dtype = 2, 96, 2, 64, BF16
    n, d = B * S, H * D
    x = round_to_dtype(normal(76, 0, (n, d)), dtype)
    ws = [round_to_dtype(normal(76, 1 + i, (d, d), std=0.05), dtype) for i in range(4)]
    up = round_to_dtype(normal(76, 9, (n, d)), dtype)

    def build():
        leaf = lambda a: Node.leaf(Layout(*a.shape), dtype, AnyBuffer.from_numpy(device, a, dtype))
        lx, (lq, lk, lv, lo) = leaf(x), [leaf(w) for w in ws]
        proj = lambda w: Node("RESHAPE", Layout(B, S, H, D), dtype, [Node("MATMUL_BT", Layout(n, d), dtype, [lx, w])])
        mask = Node.leaf(Layout(1), dtype, AnyBuffer.create(dtype, device, 1, fill=0.0))
        attn = Node("FLASH_ATTN", Layout(B, H, S, D), dtype, [proj(lq), proj(lk), proj(lv), mask],
                    {"scale": 0.125, "is_causal": True, "has_bias": False})
        o = Node("GETTUPLE", Layout(B, H, S, D), dtype, [attn], {"index": 0})
        tr = Node("TRANSPOSE", Layout(B, H, S, D).transpose(1, 2), dtype, [o], {"dim0": 1, "dim1": 2})
        ctx = Node("RESHAPE", Layout(n, d), dtype, [Node("CONTIGUOUS", Layout(B, S, H, D), dtype, [tr])])
        y = Node("MATMUL_BT", Layout(n, d), dtype, [ctx, lo])
        grads = R.gradient(y, leaf(up), [lx, lq, lk, lv, lo])
        return [y] + grads

    plain = [b.to_numpy() for b in evaluate_many(build(), device)]
    roots = Simplifier(GPU_REWRITES()).run_many(build())
    fused = [b.to_numpy() for b in evaluate_many(roots, device)]
    for a, b, name in zip(fused, plain, ("y", "dx", "dwq", "dwk", "dwv", "dwo")):
        np.testing.assert_array_equal(a, b, err_msg=name)
    counts = _op_counts(roots)
    assert "CONTIGUOUS" not in counts and "TRANSPOSE" not in counts, counts
    assert "ADD" not in counts, counts
    from mograd_amd.runtime import _toposort
    nodes = _toposort(Node("SINK", Layout(1), F32, list(roots)))
    assert all(nd.attrs().get("layout") == "bshd" for nd in nodes if nd.op_type in ("FLASH_ATTN", "FLASH_ATTN_GRAD"))
    assert sum(1 for nd in nodes if nd.op_type == "LINEAR_GRAD" and nd.attrs().get("accumulate")) == 2


def test_rewrite_rules_on_graph_structure():
    # no GPU: patterns, refusal when the folded tensor has another reader, redirection of the other
    # selectors of a refitted multi-output node
    from mograd_amd.rewrites import GPU_REWRITES, Simplifier

    x, w, b, r = Node.leaf(Layout(4, 8)), Node.leaf(Layout(6, 8)), Node.leaf(Layout(6)), Node.leaf(Layout(4, 6))
    mm = Node("MATMUL_BT", Layout(4, 6), F32, [x, w])
    out = Simplifier(GPU_REWRITES()).run(Node("ADD", Layout(4, 6), F32, [r, mm]))
    assert out.op_type == "MATMUL_BT_ADD" and out.srcs == [x, w, r]
    # the product has a second reader: it must stay a node of its own
    both = Simplifier(GPU_REWRITES()).run_many([Node("ADD", Layout(4, 6), F32, [mm, r]), mm])
    assert both[0].op_type == "ADD" and both[1] is mm
    act = Node("RELU", Layout(4, 6), F32, [Node("MATMUL_BIAS_BT", Layout(4, 6), F32, [x, w, b])])
    assert Simplifier(GPU_REWRITES()).run(act).op_type == "MATMUL_BIAS_RELU_BT"
    # RELU_GRAD folded into the LINEAR_GRAD that reads the ReLU's output: dW's selector follows
    y = Node("RELU", Layout(4, 8), F32, [x])
    z = Node("MATMUL_BT", Layout(4, 6), F32, [y, w])
    dx, dw = R.gradient(z, Node.leaf(Layout(4, 6)), [x, w])
    assert dx.op_type == "RELU_GRAD"
    dx2, dw2 = Simplifier(GPU_REWRITES()).run_many([dx, dw])
    assert dx2.op_type == "GETTUPLE" and dx2.src(0).op_type == "LINEAR_GRAD" and dx2.src(0).attrs()["relu_mask"] is True
    assert dw2.src(0) is dx2.src(0), "dW reads the refitted node, not a second copy of the product"
    # a LayerNorm that feeds a Linear layer on a skip connection: h2 = h + Linear(LayerNorm(h)).  The
    # LayerNorm's backward and the ADD of the skip connection's share fold into the layer's backward;
    # dW and db move to the new node's outputs 3 and 4, and the product is not computed twice.
    hh, gam, bet, wl, bl = (Node.leaf(Layout(*sh)) for sh in ((4, 8), (8,), (8,), (6, 8), (6,)))
    ln = Node("LAYER_NORM_STATS", Layout(4, 8), F32, [hh, gam, bet], {"eps": 1e-5})
    xn = Node("GETTUPLE", Layout(4, 8), F32, [ln], {"index": 0})
    lin_out = Node("MATMUL_BIAS_BT", Layout(4, 6), F32, [xn, wl, bl])
    w_back = Node.leaf(Layout(8, 6))
    h2 = Node("ADD", Layout(4, 8), F32, [hh, Node("MATMUL_BT", Layout(4, 8), F32, [lin_out, w_back])])
    grads = R.gradient(h2, Node.leaf(Layout(4, 8)), [hh, gam, bet, wl, bl])
    dh, dgam, dbet, dwl, dbl = Simplifier(GPU_REWRITES()).run_many(grads)
    fused = dh.src(0)
    assert dh.op_type == "GETTUPLE" and fused.op_type == "LINEAR_LAYER_NORM_GRAD" and fused.attrs()["accumulate"] is True
    assert len(fused.srcs) == 8 and fused.srcs[1] is xn and fused.srcs[2] is wl and fused.srcs[3] is hh
    for sel, index in ((dh, 0), (dgam, 1), (dbet, 2), (dwl, 3), (dbl, 4)):
        assert sel.op_type == "GETTUPLE" and sel.src(0) is fused and sel.attrs()["index"] == index
    assert _op_counts([dh, dgam, dbet, dwl, dbl]).get("LINEAR_GRAD") == 1  # only the one of w_back is left
    # dX of the product has a second reader: the two nodes stay apart
    grads = R.gradient(h2, Node.leaf(Layout(4, 8)), [hh, xn])
    kept = Simplifier(GPU_REWRITES()).run_many(grads)
    assert kept[0].src(0).op_type == "LAYER_NORM_STATS_GRAD_ADD" and kept[1].src(0).op_type == "LINEAR_GRAD"
    # the gradient rules added for residual and embedding graphs
    emb, idx = Node.leaf(Layout(10, 8)), Node.leaf(Layout(4), I32)
    h = Node("GATHER", Layout(4, 8), F32, [emb, idx])
    s2 = Node("ADD", Layout(4, 8), F32, [h, Node("CONTIGUOUS", Layout(4, 8), F32, [h])])
    (g,) = R.gradient(s2, Node.leaf(Layout(4, 8)), [emb])
    assert g.op_type == "SCATTER_ADD" and g.src(0) is idx and g.src(1).op_type == "ADD"
    c = Node("CAST", Layout(4, 8), BF16, [x])
    (gc,) = R.gradient(c, Node.leaf(Layout(4, 8), BF16), [x])
    assert gc.op_type == "CAST" and gc.dtype() == F32
