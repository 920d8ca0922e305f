"""CPU oracle (numpy, float64) for mograd's backward hot path.

TEST INFRASTRUCTURE ONLY.  This module restates the reference's arithmetic on the
CPU so that the HIP kernels can be checked against it.  Nothing in the shipped
library imports it; only tests, the smoke check and the benchmark's CPU-baseline
leg do.

Every function cites the reference lines it restates (paths relative to the
reference checkout).  All functions take array-likes, compute in float64 unless
a dtype is passed, and return numpy arrays.

Pinning (what makes each function trustworthy without running the reference):
  layer_norm_fwd        goldens tests/test_nn.mojo:283-324, torch.layer_norm (f64)
  layer_norm_bwd        goldens tests/test_grad.mojo:776-856, torch autograd (f64),
                        invariants sum(dx)=0, sum(dx*xhat)=0 for gamma=1
  cross_entropy         goldens tests/test_ops.mojo:155-183,
                        tests/test_non_contiguous.mojo:275-299, torch CE (f64)
  cross_entropy_grad    golden tests/test_non_contiguous.mojo:302-310, row sums = 0
                        (tests/test_grad.mojo:432-446), torch autograd (f64)
  sdpa_fwd / sdpa_bwd   closed forms tests/test_ops.mojo:903-946,
                        tests/test_grad.mojo:1001-1023, brute-force loop twin
                        (sdpa_*_loops), torch SDPA autograd (f64)
  matmul* / sum_axis    numpy BLAS identities, finite differences
  gather / scatter_add  index arithmetic by definition; adjoint identity
                        <gather(W, i), Y> = <W, scatter_add(i, Y)>; torch index_add_
  tiny_transformer_step torch autograd (f64) on the same model, finite differences
  adam_step / sgd_step  torch.optim.Adam / AdamW / SGD over several steps (f64)
  softmax / softmax_grad torch.softmax and its autograd (f64), rows sum to 1 / to 0
  argmax_axis           numpy.argmax on NaN-free input (first occurrence), hand cases
  round_class           tests/test_memory.mojo:18-30 (1000 -> 1024, 1025 -> 1152)
All of the above are exercised in tests/test_oracle.py.
"""
from __future__ import annotations

import math

import numpy as np

F64 = np.float64


# --------------------------------------------------------------------------- #
# LayerNorm
# --------------------------------------------------------------------------- #


def layer_norm_stats(x, eps):
    """mean and rstd per row.

    mograd/runtime/gpu/kernels/normalization.mojo:126-137 — mu = sum(x)/n,
    rstd = rsqrt(max(sum(x^2)/n - mu^2, 0) + eps) (biased variance, clamped).
    """
    x = np.asarray(x, dtype=F64)
    n = x.shape[-1]
    mu = x.sum(axis=-1, keepdims=True) / n
    var = np.maximum((x * x).sum(axis=-1, keepdims=True) / n - mu * mu, 0.0)
    rstd = 1.0 / np.sqrt(var + eps)
    return mu, rstd


def layer_norm_fwd(x, gamma, beta, eps=1e-5):
    """y = (x - mu) * rstd * gamma + beta over the last axis.

    mograd/runtime/gpu/kernels/normalization.mojo:23-59 (wraps MAX layer_norm);
    formula per mograd/nn/modules/normalization.mojo:17-27 (biased variance).
    """
    x = np.asarray(x, dtype=F64)
    mu, rstd = layer_norm_stats(x, eps)
    return (x - mu) * rstd * np.asarray(gamma, dtype=F64) + np.asarray(beta, dtype=F64)


def layer_norm_bwd(dy, x, gamma, eps=1e-5):
    """(dx, dgamma, dbeta) for y = LN(x) * gamma + beta.

    mograd/runtime/gpu/kernels/normalization.mojo:139-170:
      xhat = (x - mu) * rstd ; c1 = sum(dy*gamma)/n ; c2 = sum(dy*gamma*xhat)/n
      dx = rstd * (dy*gamma - c1 - xhat*c2)
      dgamma = sum_rows(dy * xhat) ; dbeta = sum_rows(dy)     (:281-303)
    rows = numel / cols, cols = last dim (dispatch.mojo:336-340).
    """
    dy = np.asarray(dy, dtype=F64)
    x = np.asarray(x, dtype=F64)
    g = np.asarray(gamma, dtype=F64)
    cols = x.shape[-1]
    x2 = x.reshape(-1, cols)
    dy2 = dy.reshape(-1, cols)
    mu, rstd = layer_norm_stats(x2, eps)
    xhat = (x2 - mu) * rstd
    dyg = dy2 * g
    c1 = dyg.sum(axis=1, keepdims=True) / cols
    c2 = (dyg * xhat).sum(axis=1, keepdims=True) / cols
    dx = rstd * (dyg - c1 - xhat * c2)
    dgamma = (dy2 * xhat).sum(axis=0)
    dbeta = dy2.sum(axis=0)
    return dx.reshape(x.shape), dgamma, dbeta


# --------------------------------------------------------------------------- #
# Softmax cross-entropy
# --------------------------------------------------------------------------- #


def _rows(a):
    a = np.asarray(a, dtype=F64)
    return a.reshape(-1, a.shape[-1])


def cross_entropy(logits, labels):
    """Mean softmax cross-entropy with DENSE labels (one-hot or soft).

    mograd/runtime/gpu/kernels/cross_entropy.mojo:35-77 — per row
    -(1/N) * sum_c label * (x - max - log(sum(exp(x - max)))), then sum_rows
    (:155-177).  N = numel / C, C = last dim (kernels/__init__.mojo:1386-1387).
    """
    x = _rows(logits)
    y = _rows(labels)
    n = x.shape[0]
    m = x.max(axis=1, keepdims=True)
    lse = np.log(np.exp(x - m).sum(axis=1, keepdims=True))
    row = -((x - m - lse) * y).sum(axis=1) / n
    return row.sum()


def cross_entropy_grad(logits, labels, upstream=1.0):
    """dlogits = (softmax(x) - label) * upstream / N.

    mograd/runtime/gpu/kernels/cross_entropy.mojo:207-241.
    """
    x = _rows(logits)
    y = _rows(labels)
    n = x.shape[0]
    m = x.max(axis=1, keepdims=True)
    e = np.exp(x - m)
    p = e / e.sum(axis=1, keepdims=True)
    out = (p - y) * (float(upstream) / n)
    return out.reshape(np.asarray(logits).shape)


def one_hot(ids, num_classes):
    """Dense one-hot rows, the form examples/mnist/train.mojo:36 feeds to CE."""
    ids = np.asarray(ids).reshape(-1).astype(np.int64)
    out = np.zeros((ids.size, num_classes), dtype=F64)
    out[np.arange(ids.size), ids] = 1.0
    return out


def cross_entropy_ids(logits, ids):
    """Integer-label form: identical to cross_entropy(logits, one_hot(ids))."""
    x = _rows(logits)
    ids = np.asarray(ids).reshape(-1).astype(np.int64)
    n = x.shape[0]
    m = x.max(axis=1)
    lse = np.log(np.exp(x - m[:, None]).sum(axis=1))
    picked = x[np.arange(n), ids]
    return (-(picked - m - lse) / n).sum()


def cross_entropy_grad_ids(logits, ids, upstream=1.0):
    """Integer-label form of cross_entropy_grad."""
    x = _rows(logits)
    ids = np.asarray(ids).reshape(-1).astype(np.int64)
    n = x.shape[0]
    m = x.max(axis=1, keepdims=True)
    e = np.exp(x - m)
    p = e / e.sum(axis=1, keepdims=True)
    p[np.arange(n), ids] -= 1.0
    return (p * (float(upstream) / n)).reshape(np.asarray(logits).shape)


# --------------------------------------------------------------------------- #
# Scaled dot-product attention.  Q, K, V, dQ, dK, dV are BSHD; O and dO are BHSD;
# mask is (B, H, S, S) additive in natural-log units; LSE is (B, H, S) natural log
# (mograd/runtime/gpu/kernels/attention/generic.mojo:29-35).
# --------------------------------------------------------------------------- #


def _scores(q, k, mask, has_mask, causal, scale):
    # q, k: (B, S, H, D) -> scores (B, H, S, S)
    s = np.einsum("bihd,bjhd->bhij", q, k) * scale
    if has_mask:
        s = s + mask
    if causal:
        S = q.shape[1]
        keep = np.tril(np.ones((S, S), dtype=bool))
        s = np.where(keep, s, -np.inf)
    return s


def sdpa_fwd(q, k, v, mask=None, causal=False, scale=None):
    """(O in BHSD, LSE natural log).  tests/kernels/attention/harness.mojo:58-109."""
    q = np.asarray(q, dtype=F64)
    k = np.asarray(k, dtype=F64)
    v = np.asarray(v, dtype=F64)
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    has_mask = mask is not None
    if has_mask:
        mask = np.asarray(mask, dtype=F64)
    s = _scores(q, k, mask, has_mask, causal, scale)
    m = s.max(axis=-1, keepdims=True)
    e = np.exp(s - m)
    denom = e.sum(axis=-1, keepdims=True)
    p = e / denom
    o = np.einsum("bhij,bjhd->bhid", p, v)
    lse = (m + np.log(denom))[..., 0]
    return o, lse


def sdpa_bwd(q, k, v, do, mask=None, causal=False, scale=None):
    """(dQ, dK, dV) all BSHD, with dO in BHSD.

    tests/kernels/attention/harness.mojo:112-175:
      P = softmax(S) ; delta_i = sum_d dO[i,d] * O[i,d] ; dP = dO V^T
      dS = P * (dP - delta) * scale ; dQ = dS K ; dK = dS^T Q ; dV = P^T dO
    """
    q = np.asarray(q, dtype=F64)
    k = np.asarray(k, dtype=F64)
    v = np.asarray(v, dtype=F64)
    do = np.asarray(do, dtype=F64)
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    has_mask = mask is not None
    if has_mask:
        mask = np.asarray(mask, dtype=F64)
    s = _scores(q, k, mask, has_mask, causal, scale)
    m = s.max(axis=-1, keepdims=True)
    e = np.exp(s - m)
    p = e / e.sum(axis=-1, keepdims=True)
    o = np.einsum("bhij,bjhd->bhid", p, v)
    delta = (do * o).sum(axis=-1, keepdims=True)
    dp = np.einsum("bhid,bjhd->bhij", do, v)
    ds = p * (dp - delta) * scale
    dq = np.einsum("bhij,bjhd->bihd", ds, k)
    dk = np.einsum("bhij,bihd->bjhd", ds, q)
    dv = np.einsum("bhij,bhid->bjhd", p, do)
    return dq, dk, dv


def sdpa_fwd_loops(q, k, v, mask, has_mask, causal, B, S, H, D, scale):
    """Scalar-loop twin of sdpa_fwd on flat lists; tiny sizes only.

    Same loop nest and index expressions as
    tests/kernels/attention/harness.mojo:82-109; used to pin the vectorised form.
    """
    out = [0.0] * (B * H * S * D)
    lse = [0.0] * (B * H * S)
    for b in range(B):
        for h in range(H):
            obase = (b * H + h) * S * D
            mbase = (b * H + h) * S * S
            for i in range(S):
                j_end = i + 1 if causal else S
                sc = [0.0] * j_end
                for j in range(j_end):
                    acc = 0.0
                    for d in range(D):
                        acc += q[((b * S + i) * H + h) * D + d] * k[((b * S + j) * H + h) * D + d]
                    acc *= scale
                    if has_mask:
                        acc += mask[mbase + i * S + j]
                    sc[j] = acc
                row_max = max(sc)
                ex = [math.exp(t - row_max) for t in sc]
                denom = sum(ex)
                for d in range(D):
                    acc = 0.0
                    for j in range(j_end):
                        acc += ex[j] * v[((b * S + j) * H + h) * D + d]
                    out[obase + i * D + d] = acc / denom
                lse[(b * H + h) * S + i] = row_max + math.log(denom)
    return out, lse


def sdpa_bwd_loops(q, k, v, dy, mask, has_mask, causal, B, S, H, D, scale):
    """Scalar-loop twin of sdpa_bwd (harness.mojo:137-175); tiny sizes only."""
    n = B * S * H * D
    dq = [0.0] * n
    dk = [0.0] * n
    dv = [0.0] * n
    for b in range(B):
        for h in range(H):
            mbase = (b * H + h) * S * S
            dyb = (b * H + h) * S * D
            for i in range(S):
                j_end = i + 1 if causal else S
                p = [0.0] * j_end
                for j in range(j_end):
                    acc = 0.0
                    for d in range(D):
                        acc += q[((b * S + i) * H + h) * D + d] * k[((b * S + j) * H + h) * D + d]
                    acc *= scale
                    if has_mask:
                        acc += mask[mbase + i * S + j]
                    p[j] = acc
                row_max = max(p)
                p = [math.exp(t - row_max) for t in p]
                denom = sum(p)
                p = [t / denom for t in p]
                delta = 0.0
                for d in range(D):
                    o_d = 0.0
                    for j in range(j_end):
                        o_d += p[j] * v[((b * S + j) * H + h) * D + d]
                    delta += dy[dyb + i * D + d] * o_d
                for j in range(j_end):
                    dp = 0.0
                    for d in range(D):
                        dp += dy[dyb + i * D + d] * v[((b * S + j) * H + h) * D + d]
                    ds = p[j] * (dp - delta) * scale
                    for d in range(D):
                        dq[((b * S + i) * H + h) * D + d] += ds * k[((b * S + j) * H + h) * D + d]
                        dk[((b * S + j) * H + h) * D + d] += ds * q[((b * S + i) * H + h) * D + d]
                        dv[((b * S + j) * H + h) * D + d] += p[j] * dy[dyb + i * D + d]
    return dq, dk, dv


# --------------------------------------------------------------------------- #
# Linear: forward and the three gradients
# --------------------------------------------------------------------------- #


def matmul_bias_bt(x, w, b=None):
    """Y = X W^T (+ b).  kernels/__init__.mojo:778-809 (bias epilogue adds b[n])."""
    y = np.asarray(x, dtype=F64) @ np.asarray(w, dtype=F64).T
    if b is not None:
        y = y + np.asarray(b, dtype=F64)
    return y


def linear_grad_x(dy, w):
    """dX = dY W.  mograd/grad.mojo:183 (`upstream.matmul(b.transpose())`, b = W^T)."""
    return np.asarray(dy, dtype=F64) @ np.asarray(w, dtype=F64)


def linear_grad_w(dy, x):
    """dW = dY^T X, shape (N, K).  mograd/grad.mojo:183,186-187 computes
    X^T dY (K, N) and views it transposed; the values are the same matrix."""
    dy2 = _rows(dy)
    x2 = _rows(x)
    return dy2.T @ x2


def linear_grad_b(dy):
    """db = column sums of dY.  mograd/grad.mojo:278-288 -> SUM(axis=0)
    (kernels/reduce.mojo:137-173)."""
    return _rows(dy).sum(axis=0)


def relu_grad(out, upstream):
    """upstream where relu output > 0, else 0.  kernels/elementwise.mojo:66-67."""
    out = np.asarray(out, dtype=F64)
    return np.where(out > 0, np.asarray(upstream, dtype=F64), 0.0)


def relu(a):
    """max(a, 0).  kernels/elementwise.mojo (relu_op)."""
    a = np.asarray(a, dtype=F64)
    return np.where(a > 0, a, 0.0)


# --------------------------------------------------------------------------- #
# Embedding lookup and its gradient
# --------------------------------------------------------------------------- #


def gather(src, indices):
    """out[..., :] = src[indices[...], :].  kernels/gather_scatter.mojo:14-38."""
    src = np.asarray(src, dtype=F64)
    idx = np.asarray(indices, dtype=np.int64)
    return src[idx]


def scatter_add(indices, values, num_rows):
    """dst[r, :] = sum of values[i, :] over i with indices[i] == r, dst zero elsewhere.
    kernels/gather_scatter.mojo:46-71 (atomic adds into a zero-filled buffer)."""
    idx = np.asarray(indices, dtype=np.int64).reshape(-1)
    vals = np.asarray(values, dtype=F64)
    vals = vals.reshape(idx.size, -1)
    dst = np.zeros((num_rows, vals.shape[1]), dtype=F64)
    for i in range(idx.size):  # plain loop: this is the definition
        dst[idx[i]] += vals[i]
    return dst


# --------------------------------------------------------------------------- #
# The char-level transformer of examples/tinyshakespear/model.mojo: forward, loss and
# every parameter gradient, composed from the functions above the way mograd/grad.mojo
# composes the gradient graph.
#   h = embed[ids]
#   per block: h = h + W_O(attn(W_Q(LN1 h), W_K(LN1 h), W_V(LN1 h), causal))
#              h = h + W2(relu(W1(LN2 h) + b1))
#   logits = lm_head(h) ; loss = mean cross-entropy
# --------------------------------------------------------------------------- #


def tiny_transformer_step(params, ids, labels, n_heads, eps=1e-5, store=None):
    """Returns (loss, grads) with grads shaped like params.

    params = {"embed": (V, d), "lm_head": (V, d), "blocks": [ {"ln1_g","ln1_b","wq","wk",
    "wv","wo" (d, d), "ln2_g","ln2_b","w1" (ff, d),"b1" (ff),"w2" (d, ff)} ... ]};
    ids, labels: (B, T) integers.  model.mojo:22-26,62-64,88-101,120-121.

    `store`, if given, is applied to every tensor an op of the graph writes to memory
    (each activation, each gradient); passing the rounding of a 16-bit storage type
    reproduces where a reduced-precision run rounds, the arithmetic staying float64.
    """
    r = (lambda a: a) if store is None else (lambda a: np.asarray(store(a), dtype=F64))
    ids = np.asarray(ids, dtype=np.int64)
    labels = np.asarray(labels, dtype=np.int64)
    B, T = ids.shape
    embed = np.asarray(params["embed"], dtype=F64)
    V, d = embed.shape
    dh = d // n_heads
    n = B * T
    h = gather(embed, ids.reshape(-1))  # (n, d)
    saved = []
    for blk in params["blocks"]:
        c = {"h_in": h}
        c["x1"] = r(layer_norm_fwd(h, blk["ln1_g"], blk["ln1_b"], eps))
        q = r(matmul_bias_bt(c["x1"], blk["wq"])).reshape(B, T, n_heads, dh)
        k = r(matmul_bias_bt(c["x1"], blk["wk"])).reshape(B, T, n_heads, dh)
        v = r(matmul_bias_bt(c["x1"], blk["wv"])).reshape(B, T, n_heads, dh)
        o, _ = sdpa_fwd(q, k, v, causal=True)  # BHSD
        o = r(o)
        c["q"], c["k"], c["v"] = q, k, v
        c["ctx"] = o.transpose(0, 2, 1, 3).reshape(n, d)
        h = r(h + r(matmul_bias_bt(c["ctx"], blk["wo"])))
        c["h_mid"] = h
        c["x2"] = r(layer_norm_fwd(h, blk["ln2_g"], blk["ln2_b"], eps))
        c["a"] = relu(r(matmul_bias_bt(c["x2"], blk["w1"], blk["b1"])))
        h = r(h + r(matmul_bias_bt(c["a"], blk["w2"])))
        saved.append(c)
    logits = r(matmul_bias_bt(h, params["lm_head"]))
    flat_labels = labels.reshape(-1)
    loss = cross_entropy_ids(logits, flat_labels)
    dlogits = r(cross_entropy_grad_ids(logits, flat_labels, 1.0))

    grads = {"lm_head": r(linear_grad_w(dlogits, h)), "blocks": []}
    dh_ = r(linear_grad_x(dlogits, params["lm_head"]))
    for blk, c in zip(reversed(params["blocks"]), reversed(saved)):
        g = {}
        # h = h_mid + W2 a
        g["w2"] = r(linear_grad_w(dh_, c["a"]))
        da = relu_grad(c["a"], r(linear_grad_x(dh_, blk["w2"])))
        g["w1"] = r(linear_grad_w(da, c["x2"]))
        g["b1"] = r(linear_grad_b(da))
        dx2 = r(linear_grad_x(da, blk["w1"]))
        dmid, dg, db = layer_norm_bwd(dx2, c["h_mid"], blk["ln2_g"], eps)
        g["ln2_g"], g["ln2_b"] = r(dg), r(db)
        dh_ = r(dh_ + r(dmid))
        # h_mid = h_in + W_O ctx
        g["wo"] = r(linear_grad_w(dh_, c["ctx"]))
        dctx = r(linear_grad_x(dh_, blk["wo"]))
        do = dctx.reshape(B, T, n_heads, dh).transpose(0, 2, 1, 3)  # BHSD
        dq, dk, dv = sdpa_bwd(c["q"], c["k"], c["v"], do, causal=True)
        dq, dk, dv = (r(t).reshape(n, d) for t in (dq, dk, dv))
        g["wq"] = r(linear_grad_w(dq, c["x1"]))
        g["wk"] = r(linear_grad_w(dk, c["x1"]))
        g["wv"] = r(linear_grad_w(dv, c["x1"]))
        dx1 = r(r(r(linear_grad_x(dq, blk["wq"])) + r(linear_grad_x(dk, blk["wk"]))) + r(linear_grad_x(dv, blk["wv"])))
        din, dg, db = layer_norm_bwd(dx1, c["h_in"], blk["ln1_g"], eps)
        g["ln1_g"], g["ln1_b"] = r(dg), r(db)
        dh_ = r(dh_ + r(din))
        grads["blocks"].insert(0, g)
    grads["embed"] = r(scatter_add(ids.reshape(-1), dh_, V))
    return float(loss), grads


# --------------------------------------------------------------------------- #
# Softmax, its gradient, argmax
# --------------------------------------------------------------------------- #


def softmax(x):
    """Row softmax over the last axis.  kernels/softmax.mojo:19-38 (wraps MAX nn.softmax)."""
    x = np.asarray(x, dtype=F64)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def softmax_grad(y, upstream):
    """y * (upstream - sum_c y * upstream).  kernels/softmax.mojo:76-98."""
    y = np.asarray(y, dtype=F64)
    up = np.asarray(upstream, dtype=F64)
    return y * (up - (y * up).sum(axis=-1, keepdims=True))


def argmax_axis(a, axis):
    """Index of the first strictly-largest value along `axis`, by the reference's loop:
    start from -inf at index 0, replace only on `v > best` (kernels/reduce.mojo:225-236).
    Ties go to the lowest index; NaN never wins."""
    a = np.moveaxis(np.asarray(a, dtype=F64), axis, -1)
    flat = a.reshape(-1, a.shape[-1])
    out = np.zeros(flat.shape[0], dtype=np.int64)
    for r in range(flat.shape[0]):
        best, idx = -np.inf, 0
        for i, v in enumerate(flat[r]):
            if v > best:
                best, idx = v, i
        out[r] = idx
    return out.reshape(a.shape[:-1])


# --------------------------------------------------------------------------- #
# Optimizer updates
# --------------------------------------------------------------------------- #


def adam_step(w, g, m, v, lr, beta1, beta2, eps, weight_decay, t, decoupled):
    """One Adam (decoupled=False) or AdamW (True) update; returns (w, m, v).
    mograd/nn/optim/adam.mojo:20-53."""
    w, g, m, v = (np.asarray(a, dtype=F64) for a in (w, g, m, v))
    bc1 = 1.0 - beta1 ** t
    bc2 = 1.0 - beta2 ** t
    if not decoupled and weight_decay > 0.0:
        g = g + w * weight_decay
    m = m * beta1 + g * (1.0 - beta1)
    v = v * beta2 + (g * g) * (1.0 - beta2)
    update = (m / bc1) / (np.sqrt(v / bc2) + eps) * lr
    if decoupled and weight_decay > 0.0:
        w = w * (1.0 - lr * weight_decay)
    return w - update, m, v


def sgd_step(w, g, lr):
    """w - g * lr.  mograd/nn/optim/sgd.mojo:33-36."""
    return np.asarray(w, dtype=F64) - np.asarray(g, dtype=F64) * lr


# --------------------------------------------------------------------------- #
# Pool size classes
# --------------------------------------------------------------------------- #


def round_class(nbytes: int) -> int:
    """mograd/memory.mojo:59-72."""
    if nbytes <= 512:
        return 512
    p = 1 << (int(nbytes).bit_length() - 1)
    if p == nbytes:
        return nbytes
    step = p // 8
    return ((nbytes + step - 1) // step) * step
