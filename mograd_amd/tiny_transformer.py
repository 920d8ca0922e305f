"""One training step (forward, loss, every parameter gradient) of the character-level
transformer in the reference's examples/tinyshakespear/model.mojo, issued as a fixed
sequence of libmograd_hip calls on one stream.

    h = embed[ids]                                             model.mojo:22-26
    per block:  h = h + W_O(attn(W_Q x, W_K x, W_V x, causal)),  x = LN1(h)   :62-64,88-101
                h = h + W2(relu(W1 x + b1)),                     x = LN2(h)   :120-121
    logits = lm_head(h);  loss = mean softmax cross-entropy over all tokens

The backward pass is the graph mograd/grad.mojo builds for that forward, with the fused
entries in place of their unfused chains: mg_linear_bwd(_fused) for every Linear (with the
ReLU gradient folded into the dX product; the Q, K and V projections are one Linear with
the stacked (3d, d) weight, so their input and weight gradients are one product each),
mg_linear_bwd_layer_norm_bwd where a LayerNorm feeds a Linear (the LayerNorm's backward rides on
the product's dX tiles and its result is added to the skip connection's gradient in place),
mg_flash_attn_bwd_packed (Q | K | V and dQ | dK | dV as one (B,T,3,H,dh) tensor each, O and
dO in the projections' (B,T,H,dh) layout, so no transposing copies),
mg_cross_entropy_fused_ids, mg_scatter_add for the embedding; in the forward the residual additions and the ReLU ride on the products
that feed them (mg_matmul_bt_add, mg_matmul_bias_relu_bt).

Mixed precision: the parameters live in one fp32 arena (master weights); each step casts
the whole arena once to the compute dtype (bf16 by default) and runs every kernel in that
dtype with fp32 accumulation.  The parameter gradients are sums of fp32 partial results
(the K ranges of a split dW, the row groups of dgamma/dbeta, the slabs of the embedding
gradient) that nothing in the backward pass reads, so the step records them on an
mg_deferred list and one launch at its end (mg_finish_deferred) writes them all, in fp32,
straight into the gradient arena: no 16-bit rounding of the weight gradients and no cast.
`deferred=False` keeps the earlier sequence (each sum where it arises, gradients rounded to
the compute dtype in an arena of their own, one cast to fp32), which the tests compare with.
All activations and temporaries are allocated once per (batch, context) shape.  This module
contains no arithmetic; there is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Dict, List, Tuple

import numpy as np

from ._lib import BF16, F32, I32, I64, DTYPE_SIZE
from .runtime import AnyBuffer, Device, MogradError

BLOCK_PARAMS = ("ln1_g", "ln1_b", "wq", "wk", "wv", "wo", "ln2_g", "ln2_b", "w1", "b1", "w2")
_ALIGN = 64  # elements: every parameter starts on a 128-byte boundary in either arena


class _Slice:
    """A parameter's place in the arenas."""

    __slots__ = ("name", "shape", "offset", "numel")

    def __init__(self, name: str, shape: Tuple[int, ...], offset: int):
        self.name, self.shape, self.offset = name, shape, offset
        self.numel = int(np.prod(shape))


class TinyTransformer:
    def __init__(self, device: Device, vocab_size: int, d_model: int, d_ff: int, n_layers: int, n_heads: int,
                 compute_dtype: int = BF16, eps: float = 1e-5, deferred: bool = True):
        if d_model % n_heads:
            raise MogradError(1, "d_model must be a multiple of n_heads")
        self.device, self.lib, self.stream = device, device.lib, device.stream
        self.V, self.d, self.ff, self.L, self.H = vocab_size, d_model, d_ff, n_layers, n_heads
        self.dh = d_model // n_heads
        self.cd = compute_dtype
        self.eps = eps
        self.deferred = deferred
        self.slices: Dict[str, _Slice] = {}
        off = 0

        def place(name, shape):
            nonlocal off
            self.slices[name] = _Slice(name, shape, off)
            off += -(-int(np.prod(shape)) // _ALIGN) * _ALIGN

        d, ff, V = d_model, d_ff, vocab_size
        place("embed", (V, d))
        block_shapes = {"ln1_g": (d,), "ln1_b": (d,), "wq": (d, d), "wk": (d, d), "wv": (d, d), "wo": (d, d),
                        "ln2_g": (d,), "ln2_b": (d,), "w1": (ff, d), "b1": (ff,), "w2": (d, ff)}
        for layer in range(n_layers):
            for name in BLOCK_PARAMS:
                if name == "wq":
                    # wq, wk, wv back to back with no padding between them: together they are
                    # the (3d, d) weight of one projection whose output is Q | K | V per token.
                    for i, part in enumerate(("wq", "wk", "wv")):
                        self.slices[f"blocks.{layer}.{part}"] = _Slice(f"blocks.{layer}.{part}", (d, d), off + i * d * d)
                    off += -(-3 * d * d // _ALIGN) * _ALIGN
                elif name not in ("wk", "wv"):
                    place(f"blocks.{layer}.{name}", block_shapes[name])
        place("lm_head", (V, d))
        self.total = off
        self.master = AnyBuffer.create(F32, device, self.total, fill=0.0)  # fp32 master weights
        self.grads = AnyBuffer.create(F32, device, self.total, fill=0.0)   # fp32 gradients, same layout
        self.work = AnyBuffer.create(self.cd, device, self.total)          # weights in the compute dtype
        self.wgrad = None if deferred else AnyBuffer.create(self.cd, device, self.total, fill=0.0)
        self.pending = C.c_void_p()
        if deferred:
            self.lib.mg_deferred_create(C.byref(self.pending))
        self._plan_key = None

    def __del__(self):
        if getattr(self, "pending", None):
            self.lib.mg_deferred_destroy(self.pending)
            self.pending = None

    # ------------------------------------------------------------------ parameters

    def load_params(self, params: dict) -> None:
        """params: {"embed", "lm_head", "blocks": [{name: array} ...]} (float arrays)."""
        host = np.zeros(self.total, dtype=np.float32)
        for name, sl in self.slices.items():
            host[sl.offset:sl.offset + sl.numel] = np.asarray(self._lookup(params, name), dtype=np.float32).reshape(-1)
        self.lib.mg_copy_to_device(self.master.data_ptr(), host.ctypes.data_as(C.c_void_p), host.nbytes, self.stream)

    @staticmethod
    def _lookup(tree: dict, name: str):
        parts = name.split(".")
        if parts[0] == "blocks":
            return tree["blocks"][int(parts[1])][parts[2]]
        return tree[name]

    def gradients(self) -> dict:
        """Downloads the fp32 gradient arena as a tree shaped like load_params' argument."""
        flat = self.grads.to_numpy()
        out = {"blocks": [dict() for _ in range(self.L)]}
        for name, sl in self.slices.items():
            g = flat[sl.offset:sl.offset + sl.numel].reshape(sl.shape).copy()
            parts = name.split(".")
            if parts[0] == "blocks":
                out["blocks"][int(parts[1])][parts[2]] = g
            else:
                out[name] = g
        return out

    def _w(self, name: str) -> C.c_void_p:
        return C.c_void_p(self.work.storage.ptr + self.slices[name].offset * DTYPE_SIZE[self.cd])

    def _g(self, name: str) -> C.c_void_p:
        """Where a parameter's gradient is written: the fp32 arena (deferred sums) or the
        compute-dtype one."""
        if self.deferred:
            return C.c_void_p(self.grads.storage.ptr + self.slices[name].offset * 4)
        return C.c_void_p(self.wgrad.storage.ptr + self.slices[name].offset * DTYPE_SIZE[self.cd])

    # ------------------------------------------------------------------ workspace

    def _plan(self, B: int, T: int) -> None:
        if self._plan_key == (B, T):
            return
        n, d, ff, V = B * T, self.d, self.ff, self.V
        dev, cd = self.device, self.cd
        new = lambda numel, dtype=cd: AnyBuffer.create(dtype, dev, numel)
        self.h = [new(n * d) for _ in range(self.L + 1)]  # residual stream entering each block, and the last
        self.saved: List[dict] = []
        for _ in range(self.L):
            self.saved.append({
                # Q | K | V per token: the (n, 3d) output of the stacked projection
                "x1": new(n * d), "qkv": new(3 * n * d),
                "lse": new(B * self.H * T, F32), "ctx": new(n * d),
                "h_mid": new(n * d), "x2": new(n * d), "a": new(n * ff),
                "mean1": new(n, F32), "rstd1": new(n, F32), "mean2": new(n, F32), "rstd2": new(n, F32),
            })
        self.tmp = {name: new(n * d) for name in ("dh", "dctx")}
        self.tmp["dqkv"] = new(3 * n * d)  # dQ | dK | dV per token
        self.tmp["da"] = new(n * ff)
        self.tmp["logits"] = new(n * V)
        self.tmp["dlogits"] = new(n * V)
        self.loss = new(1)
        self._plan_key = (B, T)

    # ------------------------------------------------------------------ one step

    def step(self, ids: AnyBuffer, labels: AnyBuffer, B: int, T: int, marks=None) -> AnyBuffer:
        """Runs forward, loss and backward for `ids`/`labels` ((B, T) int32 or int64 device
        buffers).  Returns the loss buffer (one element, compute dtype); the fp32 gradients
        are in `self.grads`.  Nothing is synchronised.  `marks`, if given, is called with
        "forward" and "backward" at the boundaries (for event timing)."""
        if ids.dtype not in (I32, I64) or labels.dtype not in (I32, I64):
            raise MogradError(1, "ids and labels must be int32 or int64")
        if ids.numel != B * T or labels.numel != B * T:
            raise MogradError(1, "ids/labels do not match (B, T)")
        self._plan(B, T)
        lib, s, cd = self.lib, self.stream, self.cd
        n, d, ff, V, H, dh = B * T, self.d, self.ff, self.V, self.H, self.dh
        scale = 1.0 / math.sqrt(dh)
        i64 = lambda *v: (C.c_int64 * len(v))(*v)

        def linear(x, w, out, N, K, bias=None):  # out(n, N) = x(n, K) w(N, K)^T (+ bias)
            if bias is None:
                lib.mg_matmul_bt(x, w, out, 1, n, N, K, K, 1, K, 1, n * K, N * K, cd, s)
            else:
                lib.mg_matmul_bias_bt(x, w, bias, out, 1, n, N, K, K, 1, K, 1, n * K, N * K, cd, s)

        P = lambda buf: buf.data_ptr()

        lib.mg_cast(P(self.master), P(self.work), self.total, F32, cd, s)

        # ---- forward
        lib.mg_gather(self._w("embed"), P(ids), P(self.h[0]), n, V, d, d, 1, ids.dtype, cd, s)
        for l in range(self.L):
            c, w = self.saved[l], (lambda name, l=l: self._w(f"blocks.{l}.{name}"))
            h_in, h_out = P(self.h[l]), P(self.h[l + 1])
            lib.mg_layer_norm_fwd_stats(h_in, w("ln1_g"), w("ln1_b"), P(c["x1"]), P(c["mean1"]), P(c["rstd1"]), n, d,
                                        self.eps, cd, s)
            # One projection with the stacked (3d, d) weight: row t of the (n, 3d) result is
            # Q | K | V of token t, i.e. (B, T, 3, H, dh), which the attention kernels read in place.
            linear(P(c["x1"]), w("wq"), P(c["qkv"]), 3 * d, d)
            # O is written (B, T, H, dh) = (n, d), the layout the output projection reads
            lib.mg_flash_attn_fwd_packed(P(c["qkv"]), None, P(c["ctx"]), P(c["lse"]), B, T, H, dh, scale, 1, 0, cd, s)
            lib.mg_matmul_bt_add(P(c["ctx"]), w("wo"), h_in, P(c["h_mid"]), 1, n, d, d, d, 1, d, 1, n * d, d * d, cd, s)
            lib.mg_layer_norm_fwd_stats(P(c["h_mid"]), w("ln2_g"), w("ln2_b"), P(c["x2"]), P(c["mean2"]),
                                        P(c["rstd2"]), n, d, self.eps, cd, s)
            lib.mg_matmul_bias_relu_bt(P(c["x2"]), w("w1"), w("b1"), P(c["a"]), 1, n, ff, d, d, 1, d, 1, n * d, ff * d, cd,
                                       s)
            lib.mg_matmul_bt_add(P(c["a"]), w("w2"), P(c["h_mid"]), h_out, 1, n, d, ff, ff, 1, ff, 1, n * ff, d * ff, cd,
                                 s)
        linear(P(self.h[self.L]), self._w("lm_head"), P(self.tmp["logits"]), V, d)
        lib.mg_cross_entropy_fused_ids(P(self.tmp["logits"]), P(labels), None, P(self.loss), P(self.tmp["dlogits"]), n,
                                       V, cd, labels.dtype, s)
        if marks:
            marks("forward")

        # ---- backward
        t = {k: P(v) for k, v in self.tmp.items()}
        if self.deferred:
            q = self.pending

            def lin_bwd(dy, x, w, dx, dw, db, N, K, accumulate=0, relu=0):
                lib.mg_linear_bwd_deferred(dy, x, w, dx, dw, db, n, N, K, accumulate, relu, cd, F32, q, s)

            def lin_ln_bwd(dy, x, w, dw, db, N, h, gam, mean, rstd, dg, dbt):  # dh += LayerNorm backward of dY W
                lib.mg_linear_bwd_layer_norm_bwd(dy, x, w, h, gam, mean, rstd, t["dh"], dw, db, dg, dbt, n, N, d, 1, cd,
                                                 F32, q, s)
        else:
            def lin_bwd(dy, x, w, dx, dw, db, N, K, accumulate=0, relu=0):
                lib.mg_linear_bwd_fused(dy, x, w, dx, dw, db, n, N, K, accumulate, relu, cd, s)

            def lin_ln_bwd(dy, x, w, dw, db, N, h, gam, mean, rstd, dg, dbt):
                lib.mg_linear_bwd_layer_norm_bwd(dy, x, w, h, gam, mean, rstd, t["dh"], dw, db, dg, dbt, n, N, d, 1, cd,
                                                 cd, None, s)

        lin_bwd(t["dlogits"], P(self.h[self.L]), self._w("lm_head"), t["dh"], self._g("lm_head"), None, V, d)
        for l in reversed(range(self.L)):
            c = self.saved[l]
            w = lambda name, l=l: self._w(f"blocks.{l}.{name}")
            g = lambda name, l=l: self._g(f"blocks.{l}.{name}")
            # h_out = h_mid + W2 a; the ReLU's gradient rides on the dX product
            lin_bwd(t["dh"], P(c["a"]), w("w2"), t["da"], g("w2"), None, d, ff, relu=1)
            # the layer's input is LayerNorm(h_mid): its backward rides on the dX tiles, dh += the result
            # (the skip connection's share is already in dh)
            lin_ln_bwd(t["da"], P(c["x2"]), w("w1"), g("w1"), g("b1"), ff, P(c["h_mid"]), w("ln2_g"), P(c["mean2"]),
                       P(c["rstd2"]), g("ln2_g"), g("ln2_b"))
            # h_mid = h_in + W_O ctx
            lin_bwd(t["dh"], P(c["ctx"]), w("wo"), t["dctx"], g("wo"), None, d, d)
            # dctx and ctx are (B, T, H, dh); dQ | dK | dV come back as one (n, 3d) tensor
            lib.mg_flash_attn_bwd_packed(t["dctx"], P(c["ctx"]), P(c["qkv"]), None, P(c["lse"]), t["dqkv"], B, T, H, dh,
                                         scale, 1, 0, cd, s)
            # gradient of the stacked projection: dx1 (n, d) and dW (3d, d) = dwq | dwk | dwv
            lin_ln_bwd(t["dqkv"], P(c["x1"]), w("wq"), g("wq"), None, 3 * d, P(self.h[l]), w("ln1_g"), P(c["mean1"]),
                       P(c["rstd1"]), g("ln1_g"), g("ln1_b"))
        if self.deferred:
            lib.mg_scatter_add_deferred(P(ids), t["dh"], self._g("embed"), n, V, d, ids.dtype, cd, F32, self.pending, s)
            lib.mg_finish_deferred(self.pending, s)
        else:
            lib.mg_scatter_add(P(ids), t["dh"], self._g("embed"), n, V, d, ids.dtype, cd, s)
            lib.mg_cast(P(self.wgrad), P(self.grads), self.total, cd, F32, s)
        if marks:
            marks("backward")
        return self.loss

    # ------------------------------------------------------------------ the same step through the rule tables

    def graph(self, ids: AnyBuffer, labels: AnyBuffer, B: int, T: int):
        """The forward pass as a node graph over the compute-dtype parameters (leaves bound to the
        slices of `self.work`), written with plain ops the way the reference's model writes it
        (examples/tinyshakespear/model.mojo): GATHER, LAYER_NORM_STATS, MATMUL_BT, ADD, RELU,
        MATMUL_BIAS_BT, attention on the stacked projection's (B, T, 3, H, dh) output, and
        cross-entropy on class ids.  Returns (loss node, {parameter name: leaf node})."""
        from .runtime import Layout, Node

        n, d, ff, V, H, dh, cd = B * T, self.d, self.ff, self.V, self.H, self.dh, self.cd
        leaves = {}

        def param(name, shape=None):
            sl = self.slices[name]
            shape = shape or sl.shape
            numel = int(np.prod(shape))
            leaf = Node.leaf(Layout(*shape), cd, AnyBuffer(self.work.storage, cd, numel, sl.offset))
            leaves[name] = leaf
            return leaf

        get = lambda node, i, layout, dtype=cd: Node("GETTUPLE", layout, dtype, [node], {"index": i})
        ids_leaf = Node.leaf(Layout(n), ids.dtype, ids)
        labels_leaf = Node.leaf(Layout(n), labels.dtype, labels)
        h = Node("GATHER", Layout(n, d), cd, [param("embed"), ids_leaf])
        for l in range(self.L):
            w = lambda name, shape=None, l=l: param(f"blocks.{l}.{name}", shape)

            def norm(x, g, b):
                ln = Node("LAYER_NORM_STATS", Layout(n, d), cd, [x, g, b], {"eps": self.eps})
                return get(ln, 0, Layout(n, d))

            x1 = norm(h, w("ln1_g"), w("ln1_b"))
            # wq | wk | wv lie back to back: one (3d, d) weight whose product is Q | K | V per token
            wqkv = w("wq", (3 * d, d))
            qkv = Node("MATMUL_BT", Layout(n, 3 * d), cd, [x1, wqkv])
            qkv5 = Node("RESHAPE", Layout(B, T, 3, H, dh), cd, [qkv])
            attn = Node("FLASH_ATTN_PACKED", Layout(B, T, H, dh), cd, [qkv5],
                        {"scale": 1.0 / math.sqrt(dh), "is_causal": True, "has_bias": False})
            ctx = Node("RESHAPE", Layout(n, d), cd, [get(attn, 0, Layout(B, T, H, dh))])
            h_mid = Node("ADD", Layout(n, d), cd, [Node("MATMUL_BT", Layout(n, d), cd, [ctx, w("wo")]), h])
            x2 = norm(h_mid, w("ln2_g"), w("ln2_b"))
            a = Node("RELU", Layout(n, ff), cd, [Node("MATMUL_BIAS_BT", Layout(n, ff), cd, [x2, w("w1"), w("b1")])])
            h = Node("ADD", Layout(n, d), cd, [Node("MATMUL_BT", Layout(n, d), cd, [a, w("w2")]), h_mid])
        logits = Node("MATMUL_BT", Layout(n, V), cd, [h, param("lm_head")])
        loss = Node("CROSS_ENTROPY_IDS", Layout(1), cd, [logits, labels_leaf])
        return loss, leaves

    def step_via_rules(self, ids: AnyBuffer, labels: AnyBuffer, B: int, T: int, deferred_sums: bool = True,
                       reuse_graph: bool = False):
        """The training step as the rule tables produce it: the forward graph of `graph`, its
        gradient graph from runtime.gradient (GRAD_RULES), both rewritten by
        Simplifier(GPU_REWRITES()) into the fused nodes, evaluated by runtime.evaluate_many.  Returns
        (loss buffer, {parameter name: gradient buffer in the compute dtype}, rewritten roots).  The
        kernels and their operands are those of `step`, so the results equal `step`'s bit for bit
        (its gradients before the cast to fp32).  The reference builds its graph anew every step
        (lazy tensors); `reuse_graph` keeps the rewritten graph of the first call with the same
        (ids, labels, B, T) and only evaluates it again."""
        from .rewrites import GPU_REWRITES, Simplifier
        from .runtime import Layout, Node, _toposort, evaluate_many, gradient

        self.lib.mg_cast(self.master.data_ptr(), self.work.data_ptr(), self.total, F32, self.cd, self.stream)
        key = (id(ids), id(labels), B, T)
        if reuse_graph and getattr(self, "_rules_graph", None) and self._rules_graph[0] == key:
            _, names, roots, interior = self._rules_graph
            for node in interior:  # forget last step's results; the leaves keep their buffers
                node.bufs = None
        else:
            loss, leaves = self.graph(ids, labels, B, T)
            names = [k for k in leaves if not k.endswith((".wk", ".wv"))]
            one = AnyBuffer.create(self.cd, self.device, 1, fill=1.0)
            grads = gradient(loss, Node.leaf(Layout(1), self.cd, one), [leaves[k] for k in names])
            roots = Simplifier(GPU_REWRITES()).run_many([loss] + grads)
            interior = [n for n in _toposort(Node("SINK", Layout(1), F32, list(roots)))[:-1] if n.op_type != "BUFFER"]
            self._rules_graph = (key, names, roots, interior) if reuse_graph else None
        bufs = evaluate_many(roots, self.device, deferred_sums=deferred_sums)
        return bufs[0], dict(zip(names, bufs[1:])), roots

    # ------------------------------------------------------------------ optimizer

    def adam_step(self, lr: float = 1e-3, beta1: float = 0.9, beta2: float = 0.999, eps: float = 1e-8,
                  weight_decay: float = 0.0, decoupled: bool = False) -> None:
        """One Adam / AdamW update of every parameter from the gradients of the last
        `step` (mograd/nn/optim/adam.mojo): a single kernel over the fp32 arenas."""
        if not hasattr(self, "adam_m"):
            self.adam_m = AnyBuffer.create(F32, self.device, self.total, fill=0.0)
            self.adam_v = AnyBuffer.create(F32, self.device, self.total, fill=0.0)
            self.adam_t = 0
        self.adam_t += 1
        self.lib.mg_adam_step(self.master.data_ptr(), self.grads.data_ptr(), self.adam_m.data_ptr(),
                              self.adam_v.data_ptr(), self.total, lr, beta1, beta2, eps, weight_decay, self.adam_t,
                              int(decoupled), self.stream)

    def parameters(self) -> dict:
        """Downloads the fp32 master weights as a tree shaped like load_params' argument."""
        flat = self.master.to_numpy()
        out = {"blocks": [dict() for _ in range(self.L)]}
        for name, sl in self.slices.items():
            a = flat[sl.offset:sl.offset + sl.numel].reshape(sl.shape).copy()
            parts = name.split(".")
            if parts[0] == "blocks":
                out["blocks"][int(parts[1])][parts[2]] = a
            else:
                out[name] = a
        return out

    # ------------------------------------------------------------------ bookkeeping

    def flops_per_step(self, B: int, T: int) -> float:
        """Matmul and attention FLOPs of one forward+backward, counted the usual way:
        2mnk per product, 3 products per Linear (forward, dX, dW), and for causal
        attention half of 4*B*H*T^2*dh forward plus 2.5 times that backward."""
        n, d, ff, V = B * T, self.d, self.ff, self.V
        per_block = 4 * d * d + 2 * d * ff
        linear = 3 * 2 * n * (self.L * per_block + V * d)
        attn_fwd = 0.5 * 4 * B * self.H * T * T * self.dh
        return linear + self.L * 3.5 * attn_fwd


def init_params(rng: np.random.Generator, vocab_size: int, d_model: int, d_ff: int, n_layers: int) -> dict:
    """Random parameters with the reference's initialisers: Embedding ~ N(0, 1)
    (nn/modules/embedding.mojo:23-29), Linear weight and bias ~ U(+-sqrt(6 / fan_in))
    (nn/modules/linear.mojo:29-47), LayerNorm gamma 1, beta 0."""
    def lin(o, i):
        b = math.sqrt(6.0 / i)
        return rng.uniform(-b, b, size=(o, i)).astype(np.float32)

    d, ff = d_model, d_ff
    blocks = []
    for _ in range(n_layers):
        blocks.append({
            "ln1_g": np.ones(d, np.float32), "ln1_b": np.zeros(d, np.float32),
            "wq": lin(d, d), "wk": lin(d, d), "wv": lin(d, d), "wo": lin(d, d),
            "ln2_g": np.ones(d, np.float32), "ln2_b": np.zeros(d, np.float32),
            "w1": lin(ff, d), "b1": rng.uniform(-math.sqrt(6.0 / d), math.sqrt(6.0 / d), ff).astype(np.float32),
            "w2": lin(d, ff),
        })
    return {"embed": rng.standard_normal((vocab_size, d)).astype(np.float32), "lm_head": lin(vocab_size, d),
            "blocks": blocks}
