"""Graph rewrites that create the fused nodes of libmograd_hip, and the pass that applies them.

The reference creates its fused nodes (MATMUL_BT, MATMUL_BIAS_BT, LAYER_NORM, FLASH_ATTN) with
`Simplifier(GPU_REWRITES())` (mograd/simplify/__init__.mojo:22-71,
mograd/runtime/gpu/rewrites.mojo:13-34): every node, sources first, is rewritten to a fixed
point by the first rule whose pattern matches, and a substitution table carries rewritten
sources to their consumers.  `Simplifier` here restates that pass; `GPU_REWRITES` holds the
rules for the fusions this library adds on top of the reference's set, the ones a transformer
training step uses:

    ADD(MATMUL_BT(a, w), r)                      -> MATMUL_BT_ADD[a, w, r]
    RELU(MATMUL_BIAS_BT(a, w, b))                -> MATMUL_BIAS_RELU_BT[a, w, b]
    RELU_GRAD(y, LINEAR_GRAD(dy, y, w)[0])       -> LINEAR_GRAD{relu_mask}(dy, y, w)[0]
    ADD(p, LINEAR_GRAD(dy, x, w)[0])             -> LINEAR_GRAD{accumulate}(dy, x, w, p)[0]
    ADD(r, LAYER_NORM_STATS_GRAD(...)[0])        -> LAYER_NORM_STATS_GRAD_ADD(..., r)[0]
    CONTIGUOUS(TRANSPOSE(FLASH_ATTN(...)[0]))    -> FLASH_ATTN{layout: bshd}(...)[0]
    FLASH_ATTN_GRAD(CONTIGUOUS(TRANSPOSE(g)), O) -> FLASH_ATTN_GRAD{layout: bshd}(g, O') when O
                                                    was rewritten to the (B, S, H, D) layout

A rule that folds a consumer into a multi-output producer (the LINEAR_GRAD and
LAYER_NORM_STATS_GRAD rules) has to change the producer for all of its consumers: the pass
records such replacements in the substitution table, so the other GETTUPLE selectors of the
producer (dW, db, dgamma, dbeta) follow, and refuses the fusion when the folded output has a
second consumer.  No arithmetic here: the fused kernels give bit for bit what the separate
ones give (include/mograd_hip.h), so a rewritten graph evaluates to the same bits.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

from .runtime import Layout, MogradError, Node, _toposort

__all__ = ["Pat", "Rule", "Simplifier", "GPU_REWRITES"]


@dataclass
class Pat:
    """An op type (None: anything) over patterns for the leading sources
    (mograd/pattern_matcher.mojo:8-60)."""

    op_type: Optional[str] = None
    srcs: Sequence["Pat"] = field(default_factory=tuple)

    def matches(self, node: Node) -> bool:
        if self.op_type is not None and node.op_type != self.op_type:
            return False
        if len(self.srcs) > len(node.srcs):
            return False
        return all(p.matches(s) for p, s in zip(self.srcs, node.srcs))


@dataclass
class Rule:
    pat: Pat
    func: Callable[[Node, "Simplifier"], Optional[Node]]
    name: str = ""


def _get0(pat: Pat) -> Pat:
    return Pat("GETTUPLE", [pat])


class Simplifier:
    """mograd/simplify/__init__.mojo:22-71: per-node fixed point over `rules`, sources first."""

    def __init__(self, rules: List[Rule]):
        self.rules = rules
        self.subst: Dict[Node, Node] = {}
        self.uses: Dict[Node, int] = {}
        self.origin: Dict[Node, Node] = {}        # rebuilt or rewritten node -> the graph's own node
        self.consumers: Dict[Node, List[Node]] = {}  # of the graph's own nodes

    # -- helpers for the rules --------------------------------------------------------------
    def single_use(self, node: Node) -> bool:
        """True when `node` (a node of the graph as it was before this node's rewrite) has at most
        one consumer: folding it into that consumer then leaves nobody without it."""
        return self.uses.get(node, 0) <= 1

    def replace(self, old: Node, new: Node) -> None:
        """Every consumer of `old` reads `new` instead (those already visited are redirected when
        the pass ends)."""
        self.subst[old] = new
        self.origin[new] = self.origin.get(old, old)

    def consumers_of(self, node: Node) -> List[Node]:
        """The consumers that `node` had in the graph as it was handed to the pass."""
        return self.consumers.get(self.origin.get(node, node), [])

    # -- the pass ---------------------------------------------------------------------------
    def _with_subst(self, node: Node) -> Node:
        if not node.srcs:
            return node
        new_srcs = [self.resolve(s) for s in node.srcs]
        if all(a is b for a, b in zip(new_srcs, node.srcs)):
            return node
        out = Node(node.op_type, node.node_layout, node.node_dtype, new_srcs, dict(node.node_attrs), node.bufs)
        self.uses[out] = self.uses.get(node, 0)
        self.origin[out] = self.origin.get(node, node)
        return out

    def resolve(self, node: Node) -> Node:
        seen = 0
        while node in self.subst:
            node = self.subst[node]
            seen += 1
            if seen > 64:
                raise MogradError(1, "Simplifier: substitutions cycled without converging")
        return node

    def run_many(self, roots: Sequence[Node]) -> List[Node]:
        sink = Node("SINK", Layout(1), 0, list(roots))
        topo = _toposort(sink)[:-1]
        self.subst, self.uses, self.origin, self.consumers = {}, {}, {}, {}
        for n in topo:
            for s_ in n.srcs:
                self.uses[s_] = self.uses.get(s_, 0) + 1
                self.consumers.setdefault(s_, []).append(n)
        for r in roots:  # a root is read by the caller
            self.uses[r] = self.uses.get(r, 0) + 1
        for node in topo:
            if node in self.subst:  # a rule that ran on another node has already replaced this one
                continue
            node_r = self._with_subst(node)
            for _ in range(64):
                progressed = False
                for rule in self.rules:
                    if not rule.pat.matches(node_r):
                        continue
                    rewritten = rule.func(node_r, self)
                    if rewritten is not None:
                        self.uses[rewritten] = self.uses.get(node_r, 0)
                        self.origin.setdefault(rewritten, self.origin.get(node_r, node_r))
                        node_r = self._with_subst(rewritten)
                        progressed = True
                        break
                if not progressed:
                    break
            else:
                raise MogradError(1, "Simplifier: rewrite rules cycled without converging")
            if node_r is not node:
                self.subst[node] = node_r
        return self._redirect(roots)

    def _redirect(self, roots: Sequence[Node]) -> List[Node]:
        """A rule may replace a node that earlier consumers already hold (the other selectors of a
        multi-output producer that was refitted for one of them): rebuilds the result so that
        every edge follows the final substitution table."""
        done: Dict[Node, Node] = {}
        stack = [(r, 0) for r in reversed(list(roots))]
        while stack:
            n, i = stack.pop()
            r = self.resolve(n)
            if r in done:
                done[n] = done[r]
                continue
            if i < len(r.srcs):
                stack.append((n, i + 1))
                child = r.srcs[i]
                if child not in done:
                    stack.append((child, 0))
                continue
            new_srcs = [done[c] for c in r.srcs]
            if all(a is b for a, b in zip(new_srcs, r.srcs)):
                out = r
            else:
                out = Node(r.op_type, r.node_layout, r.node_dtype, new_srcs, dict(r.node_attrs), r.bufs)
            done[r] = out
            done[n] = out
        return [done[r] for r in roots]

    def run(self, root: Node) -> Node:
        return self.run_many([root])[0]


# --------------------------------------------------------------------------- #
# The rules
# --------------------------------------------------------------------------- #


def _same_shape(a: Node, b: Node) -> bool:
    return a.layout().shape() == b.layout().shape()


def fuse_matmul_add(node: Node, sim: Simplifier) -> Optional[Node]:
    """ADD(MATMUL_BT(a, w), r) in either operand order -> MATMUL_BT_ADD[a, w, r]."""
    for mm, other in ((node.src(0), node.src(1)), (node.src(1), node.src(0))):
        if mm.op_type == "MATMUL_BT" and sim.single_use(mm) and _same_shape(mm, other) and mm.dtype() == other.dtype():
            return Node("MATMUL_BT_ADD", mm.layout(), node.dtype(), [mm.src(0), mm.src(1), other])
    return None


def fuse_matmul_bias_relu(node: Node, sim: Simplifier) -> Optional[Node]:
    """RELU(MATMUL_BIAS_BT(a, w, b)) -> MATMUL_BIAS_RELU_BT[a, w, b]."""
    mm = node.src(0)
    if not sim.single_use(mm):
        return None
    return Node("MATMUL_BIAS_RELU_BT", mm.layout(), node.dtype(), list(mm.srcs))


def _refit(producer: Node, op_type: str, srcs: List[Node], attrs: dict, sim: Simplifier) -> Node:
    """The multi-output `producer` with another op type / sources / attributes; every selector of
    the old one is redirected to the new one."""
    new = Node(op_type, producer.node_layout, producer.node_dtype, srcs, attrs)
    sim.replace(producer, new)
    return new


def fuse_relu_grad_into_linear_grad(node: Node, sim: Simplifier) -> Optional[Node]:
    """RELU_GRAD(y, GETTUPLE0(LINEAR_GRAD(dy, y, w))) -> GETTUPLE0(LINEAR_GRAD{relu_mask}(dy, y, w)): the
    product's input is the ReLU's own output, so the mask is the tensor the kernel already reads."""
    y, sel = node.src(0), node.src(1)
    lin = sel.src(0)
    if int(sel.attrs().get("index", -1)) != 0 or lin.src(1) is not y or not sim.single_use(sel):
        return None
    if lin.attrs().get("relu_mask") or lin.attrs().get("accumulate"):
        return None
    new = _refit(lin, "LINEAR_GRAD", list(lin.srcs), {**lin.attrs(), "relu_mask": True}, sim)
    return Node("GETTUPLE", sel.node_layout, sel.node_dtype, [new], {"index": 0})


def fuse_add_into_linear_grad(node: Node, sim: Simplifier) -> Optional[Node]:
    """ADD(p, GETTUPLE0(LINEAR_GRAD(dy, x, w))) -> GETTUPLE0(LINEAR_GRAD{accumulate}(dy, x, w, p))."""
    for sel, other in ((node.src(0), node.src(1)), (node.src(1), node.src(0))):
        if sel.op_type != "GETTUPLE" or sel.src(0).op_type != "LINEAR_GRAD" or int(sel.attrs().get("index", -1)) != 0:
            continue
        lin = sel.src(0)
        if lin.attrs().get("accumulate") or not sim.single_use(sel) or not _same_shape(sel, other):
            continue
        if other.dtype() != sel.dtype() or lin in _toposort(other):  # `other` must not depend on the product
            continue
        new = _refit(lin, "LINEAR_GRAD", list(lin.srcs) + [other], {**lin.attrs(), "accumulate": True}, sim)
        return Node("GETTUPLE", sel.node_layout, sel.node_dtype, [new], {"index": 0})
    return None


def fuse_add_into_layer_norm_grad(node: Node, sim: Simplifier) -> Optional[Node]:
    """ADD(r, GETTUPLE0(LAYER_NORM_STATS_GRAD(dy, x, g, mean, rstd))) -> GETTUPLE0(LAYER_NORM_STATS_GRAD_ADD(.., r))."""
    for sel, other in ((node.src(0), node.src(1)), (node.src(1), node.src(0))):
        if sel.op_type != "GETTUPLE" or sel.src(0).op_type != "LAYER_NORM_STATS_GRAD":
            continue
        ln = sel.src(0)
        if int(sel.attrs().get("index", -1)) != 0 or not sim.single_use(sel) or not _same_shape(sel, other):
            continue
        if other.dtype() != sel.dtype() or ln in _toposort(other):
            continue
        new = _refit(ln, "LAYER_NORM_STATS_GRAD_ADD", list(ln.srcs) + [other], dict(ln.attrs()), sim)
        return Node("GETTUPLE", sel.node_layout, sel.node_dtype, [new], {"index": 0})
    return None


def fuse_linear_grad_into_layer_norm_grad(node: Node, sim: Simplifier) -> Optional[Node]:
    """LAYER_NORM_STATS_GRAD(GETTUPLE0(LINEAR_GRAD(dy, x, w)), h, g, mean, rstd) ->
    LINEAR_LAYER_NORM_GRAD[dy, x, w, h, g, mean, rstd] with outputs [dh, dgamma, dbeta, dW, db]: the input
    gradient of a Linear layer that only the backward of the LayerNorm feeding the layer reads.  The
    LayerNorm node's selectors keep their indices; the product's dW and db selectors move to 3 and 4."""
    sel = node.src(0)
    if sel.op_type != "GETTUPLE" or int(sel.attrs().get("index", -1)) != 0 or sel.src(0).op_type != "LINEAR_GRAD":
        return None
    lin = sel.src(0)
    if lin.attrs().get("relu_mask") or lin.attrs().get("accumulate") or not sim.single_use(sel):
        return None
    if node.src(1).layout().numel() != sel.layout().numel() or node.dtype() != lin.dtype():
        return None
    attrs = {"has_bias": bool(lin.attrs().get("has_bias", True))}
    srcs = list(lin.srcs[:3]) + list(node.srcs[1:5])
    if node.op_type == "LAYER_NORM_STATS_GRAD_ADD":
        srcs.append(node.src(5))
        attrs["accumulate"] = True
    new = Node("LINEAR_LAYER_NORM_GRAD", node.node_layout, node.node_dtype, srcs, attrs)
    for c in sim.consumers_of(lin):  # dW and db of the product now come from the new node
        index = int(c.attrs().get("index", -1)) if c.op_type == "GETTUPLE" else -1
        if index in (1, 2):
            moved = Node("GETTUPLE", c.node_layout, c.node_dtype, [new], {"index": index + 2})
            sim.replace(sim.resolve(c), moved)
    return new


def fuse_add_into_linear_layer_norm_grad(node: Node, sim: Simplifier) -> Optional[Node]:
    """ADD(r, GETTUPLE0(LINEAR_LAYER_NORM_GRAD(..))) -> GETTUPLE0(LINEAR_LAYER_NORM_GRAD{accumulate}(.., r))."""
    for sel, other in ((node.src(0), node.src(1)), (node.src(1), node.src(0))):
        if sel.op_type != "GETTUPLE" or sel.src(0).op_type != "LINEAR_LAYER_NORM_GRAD":
            continue
        fused = sel.src(0)
        if int(sel.attrs().get("index", -1)) != 0 or fused.attrs().get("accumulate") or not sim.single_use(sel):
            continue
        if not _same_shape(sel, other) or other.dtype() != sel.dtype() or fused in _toposort(other):
            continue
        new = _refit(fused, "LINEAR_LAYER_NORM_GRAD", list(fused.srcs) + [other], {**fused.attrs(), "accumulate": True}, sim)
        return Node("GETTUPLE", sel.node_layout, sel.node_dtype, [new], {"index": 0})
    return None


def _is_bhsd_to_bshd(tr: Node) -> bool:
    d0, d1 = int(tr.attrs().get("dim0", -2)) % 4, int(tr.attrs().get("dim1", -1)) % 4
    return tr.layout().rank() == 4 and {d0, d1} == {1, 2}


def fuse_attention_output_layout(node: Node, sim: Simplifier) -> Optional[Node]:
    """CONTIGUOUS(TRANSPOSE{1,2}(GETTUPLE0(FLASH_ATTN(q, k, v, mask)))) -> GETTUPLE0(FLASH_ATTN{layout: bshd}):
    the copy the reference's model makes after attention (examples/tinyshakespear/model.mojo:104)
    disappears into the kernel's store.  Only when O has no other reader than this copy and the
    backward node, which is rewritten along (fuse_attention_grad_layout)."""
    tr = node.src(0)
    sel = tr.src(0)
    attn = sel.src(0)
    if not _is_bhsd_to_bshd(tr) or int(sel.attrs().get("index", -1)) != 0 or attn.attrs().get("layout") == "bshd":
        return None
    for o_sel in sim.consumers_of(attn):  # every reader of O: this copy, or the backward node's O operand
        if o_sel.op_type != "GETTUPLE" or int(o_sel.attrs().get("index", -1)) != 0:
            continue
        for c in sim.consumers.get(o_sel, []):
            copy_chain = (c.op_type == "TRANSPOSE" and _is_bhsd_to_bshd(c) and
                          all(cc.op_type == "CONTIGUOUS" for cc in sim.consumers.get(c, [])))
            if not (copy_chain or (c.op_type == "FLASH_ATTN_GRAD" and c.src(1) is o_sel)):
                return None
    B, H, S, D = sel.layout().shape()
    new = _refit(attn, "FLASH_ATTN", list(attn.srcs), {**attn.attrs(), "layout": "bshd"}, sim)
    new.node_layout = Layout(B, S, H, D)
    return Node("GETTUPLE", Layout(B, S, H, D), sel.node_dtype, [new], {"index": 0})


def fuse_attention_grad_layout(node: Node, sim: Simplifier) -> Optional[Node]:
    """FLASH_ATTN_GRAD whose O comes from a FLASH_ATTN{layout: bshd}: dO must be (B, S, H, D) too.  The
    gradient graph hands it over as CONTIGUOUS(TRANSPOSE{1,2}(g)) with g the gradient of the
    (B, S, H, D) copy: g itself is the operand."""
    if node.attrs().get("layout") == "bshd":
        return None
    o_sel = node.src(1)
    if o_sel.op_type != "GETTUPLE" or sim.resolve(o_sel.src(0)).attrs().get("layout") != "bshd":
        return None
    d_o = node.src(0)
    if d_o.op_type == "CONTIGUOUS" and d_o.src(0).op_type == "TRANSPOSE" and _is_bhsd_to_bshd(d_o.src(0)):
        g = d_o.src(0).src(0)
    else:  # any other gradient: lay it out (B, S, H, D) with one copy
        B, H, S, D = d_o.layout().shape()
        tr = Node("TRANSPOSE", d_o.layout().transpose(1, 2), d_o.dtype(), [d_o], {"dim0": 1, "dim1": 2})
        g = Node("CONTIGUOUS", Layout(B, S, H, D), d_o.dtype(), [tr])
    if not g.layout().is_contiguous():
        g = Node("CONTIGUOUS", g.layout().as_contiguous(), g.dtype(), [g])
    return _refit(node, "FLASH_ATTN_GRAD", [g] + list(node.srcs[1:]), {**node.attrs(), "layout": "bshd"}, sim)


def GPU_REWRITES() -> List[Rule]:
    """The fusions of a transformer training step, in matching priority."""
    get0 = lambda op: _get0(Pat(op))
    return [
        Rule(Pat("RELU", [Pat("MATMUL_BIAS_BT")]), fuse_matmul_bias_relu, "fuse_matmul_bias_relu"),
        Rule(Pat("RELU_GRAD", [Pat(), get0("LINEAR_GRAD")]), fuse_relu_grad_into_linear_grad,
             "fuse_relu_grad_into_linear_grad"),
        Rule(Pat("CONTIGUOUS", [Pat("TRANSPOSE", [get0("FLASH_ATTN")])]), fuse_attention_output_layout,
             "fuse_attention_output_layout"),
        Rule(Pat("FLASH_ATTN_GRAD"), fuse_attention_grad_layout, "fuse_attention_grad_layout"),
        Rule(Pat("LAYER_NORM_STATS_GRAD", [get0("LINEAR_GRAD")]), fuse_linear_grad_into_layer_norm_grad,
             "fuse_linear_grad_into_layer_norm_grad"),
        Rule(Pat("LAYER_NORM_STATS_GRAD_ADD", [get0("LINEAR_GRAD")]), fuse_linear_grad_into_layer_norm_grad,
             "fuse_linear_grad_into_layer_norm_grad"),
        Rule(Pat("ADD"), fuse_matmul_add, "fuse_matmul_add"),
        Rule(Pat("ADD"), fuse_add_into_layer_norm_grad, "fuse_add_into_layer_norm_grad"),
        Rule(Pat("ADD"), fuse_add_into_linear_layer_norm_grad, "fuse_add_into_linear_layer_norm_grad"),
        Rule(Pat("ADD"), fuse_add_into_linear_grad, "fuse_add_into_linear_grad"),
    ]
