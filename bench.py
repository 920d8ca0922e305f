#!/usr/bin/env python3
"""Benchmark of the backward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = LayerNorm forward + backward on fp32 (2048, 4096) and fused softmax
cross-entropy forward + backward on fp32 logits (8192, 50304) with int32 labels, all
inputs resident in HBM before the timed region.  Prints ONE JSON line:
  value/ms_per_step   wall time per step (K steps between two stream synchronisations)
  roofline            the dominant kernel (cross-entropy rows kernel): algorithmic bytes
                      per launch / mean launch duration from HIP events on the stream
                      the kernel runs on, against the 8 TB/s HBM peak
  kernels             the same for every kernel of the step
  cpu_baseline        the C restatement of the reference's arithmetic (oracle/), timed on
                      this host's cores on a bounded sample of the same workload
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0

LN_ROWS, LN_COLS = 2048, 4096
CE_ROWS, CE_COLS = 8192, 50304

# Algorithmic bytes per launch: what any implementation must move.
LN_FWD_BYTES = 2 * LN_ROWS * LN_COLS * 4 + 2 * LN_COLS * 4            # x, y, gamma, beta
LN_BWD_BYTES = 3 * LN_ROWS * LN_COLS * 4 + 3 * LN_COLS * 4            # dy, x, dx, gamma, dgamma, dbeta
CE_FUSED_BYTES = 2 * CE_ROWS * CE_COLS * 4 + CE_ROWS * 4 + 4          # logits, dlogits, labels, loss

def _measured_traffic(key: str):
    """HBM bytes per launch of one kernel, from the counter figures committed beside the
    profiles (profiles/hbm_traffic.json: per-dispatch means of FETCH_SIZE and WRITE_SIZE in
    KiB from two `rocprofv3 --pmc` runs of this script, and what each counter reads per true
    KiB for the plain copy of known size that the ln_ce workload performs).  None when the
    file has no such entry."""
    try:
        with open(ROOT / "profiles" / "hbm_traffic.json") as f:
            entry = json.load(f).get(key)
    except (OSError, ValueError):
        return None
    if not entry:
        return None
    return int((entry["fetch_kib"] / entry["fetch_factor"] + entry["write_kib"] / entry["write_factor"]) * 1024)


def _trace_kernel_us(key: str):
    """Average duration in microseconds of one kernel in the committed rocprofv3 kernel trace of
    this script (profiles/kernel_times.json, written from the trace's stats), or None."""
    try:
        with open(ROOT / "profiles" / "kernel_times.json") as f:
            entry = json.load(f).get(key)
    except (OSError, ValueError):
        return None
    return float(entry["avg_us"]) if entry else None


def _rng(config: int, tensor: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(1000 * config + tensor))


def _best_ms(fn, reps: int = 3) -> float:
    """Host leg timing: one untimed warm-up call (page faults, thread pool start-up), then the
    best of `reps` calls, in milliseconds."""
    fn()
    best = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
    return best * 1e3


class EventTimer:
    """Mean duration of a callable's device work, from HIP event pairs recorded on the
    library's stream around each call."""

    def __init__(self, device, n: int):
        self.dev = device
        self.lib = device.lib
        self.starts = [C.c_void_p() for _ in range(n)]
        self.stops = [C.c_void_p() for _ in range(n)]
        for e in self.starts + self.stops:
            self.lib.mg_event_create(C.byref(e))

    def run(self, fn, iters: int):
        assert iters <= len(self.starts)
        for i in range(iters):
            self.lib.mg_event_record(self.starts[i], self.dev.stream)
            fn(i)
            self.lib.mg_event_record(self.stops[i], self.dev.stream)
        self.dev.synchronize()
        ms = C.c_float()
        out = []
        for i in range(iters):
            self.lib.mg_event_elapsed_ms(self.starts[i], self.stops[i], C.byref(ms))
            out.append(ms.value)
        return out

    def close(self):
        for e in self.starts + self.stops:
            self.lib.mg_event_destroy(e)


def cpu_baseline(sample_ce_rows: int = 256):
    """Times the C restatement (oracle/oracle_c.c) on this host: LayerNorm at full size,
    cross-entropy on `sample_ce_rows` rows scaled to 8192."""
    import subprocess

    so = ROOT / "oracle" / "liboracle_c.so"
    if not so.exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    orc = C.CDLL(str(so))
    orc.orc_num_threads.restype = C.c_int
    orc.orc_cross_entropy_f32.restype = C.c_float
    cores = int(orc.orc_num_threads())
    p = lambda a: a.ctypes.data_as(C.c_void_p)  # noqa: E731
    L = C.c_int64

    x = _rng(2, 0).standard_normal((LN_ROWS, LN_COLS), dtype=np.float32)
    g = _rng(2, 1).uniform(0.5, 1.5, LN_COLS).astype(np.float32)
    b = (_rng(2, 2).standard_normal(LN_COLS) * 0.1).astype(np.float32)
    dy = _rng(2, 3).standard_normal((LN_ROWS, LN_COLS), dtype=np.float32)
    y, dx = np.empty_like(x), np.empty_like(x)
    dg, db = np.empty_like(g), np.empty_like(g)

    def ln():
        orc.orc_layer_norm_fwd_f32(p(x), p(g), p(b), p(y), L(LN_ROWS), L(LN_COLS), C.c_float(1e-5))
        orc.orc_layer_norm_bwd_f32(p(dy), p(x), p(g), p(dx), p(dg), p(db), L(LN_ROWS), L(LN_COLS), C.c_float(1e-5),
                                   L(256))

    n = sample_ce_rows
    logits = (_rng(2, 10).standard_normal((n, CE_COLS), dtype=np.float32) * 2.0)
    ids = _rng(2, 11).integers(0, CE_COLS, n).astype(np.int32)
    up = np.ones(1, np.float32)
    dlogits = np.empty_like(logits)

    onehot = np.zeros((n, CE_COLS), np.float32)
    onehot[np.arange(n), ids] = 1.0

    def ce_dense():
        # the reference's structure: forward and gradient as separate passes, each re-deriving
        # the row maximum and the sum of exponentials, labels dense (one-hot rows)
        orc.orc_cross_entropy_f32(p(logits), p(onehot), L(n), L(CE_COLS))
        orc.orc_cross_entropy_grad_f32(p(logits), p(onehot), p(up), p(dlogits), L(n), L(CE_COLS))

    def ce_ids():
        # the work the GPU leg does: class ids, loss and gradient (two passes over the logits here)
        orc.orc_cross_entropy_ids_f32(p(logits), p(ids), L(n), L(CE_COLS))
        orc.orc_cross_entropy_grad_ids_f32(p(logits), p(ids), p(up), p(dlogits), L(n), L(CE_COLS))

    orc.orc_cross_entropy_ids_f32.restype = C.c_float
    ln_ms = _best_ms(ln, 5)
    ce_ids_ms = _best_ms(ce_ids, 3) * (CE_ROWS / n)
    ce_dense_ms = _best_ms(ce_dense, 3) * (CE_ROWS / n)
    return {
        "value": round(ln_ms + ce_ids_ms, 3),
        "unit": "ms",
        "cores": cores,
        "kind": "port",
        "sample": f"LayerNorm fwd+bwd full (2048x4096) {ln_ms:.2f} ms; cross-entropy loss and gradient on class ids (the GPU leg's "
                  f"inputs) on {n} of 8192 rows scaled x{CE_ROWS // n} = {ce_ids_ms:.1f} ms; best of 3-5 runs after a warm-up, "
                  f"OpenMP on {cores} threads",
        # the reference's own form of the same loss: dense one-hot labels (another 1.65 GB stream),
        # forward and gradient as separate passes
        "dense_label_form_ms": round(ln_ms + ce_dense_ms, 3),
        "dense_label_form": f"cross-entropy with dense one-hot labels, forward and gradient as separate passes: {ce_dense_ms:.1f} ms",
    }


MFMA_F32_PEAK_TFLOPS = 157.3
MFMA_BF16_PEAK_TFLOPS = 2500.0


def _orc():
    import subprocess

    so = ROOT / "oracle" / "liboracle_c.so"
    if not so.exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    orc = C.CDLL(str(so))
    orc.orc_num_threads.restype = C.c_int
    return orc


def _time_steps(dev, step, warmup, steps):
    for i in range(warmup):
        step(i)
    dev.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(warmup + i)
    dev.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def _kernel_table(dev, entries, iters):
    """entries: (name, fn, work, unit) with unit 'B' (bytes, HBM bound) or 'F' (flops, MFMA
    bound, against `peak` TFLOP/s given as a 5th element)."""
    timer = EventTimer(dev, iters)
    out = []
    for name, fn, work, unit, peak in entries:
        fn(0)
        dev.synchronize()
        ts = timer.run(fn, iters)
        mean_ms = float(np.mean(ts))
        row = {"name": name, "mean_ms": round(mean_ms, 5), "median_ms": round(float(np.median(ts)), 5)}
        if unit == "B":
            gbs = work / (mean_ms * 1e-3) / 1e9
            row.update({"algorithmic_bytes": work, "achieved_GBps": round(gbs, 1),
                        "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)})
        else:
            tf = work / (mean_ms * 1e-3) / 1e12
            row.update({"algorithmic_flops": work, "achieved_TFLOPs": round(tf, 1), "peak_TFLOPs": peak,
                        "frac_of_mfma_peak": round(tf / peak, 4)})
        out.append(row)
    timer.close()
    return out


# --------------------------------------------------------------------------- #
# Sanity checks before timing: a few sampled rows of each workload's outputs
# against plain float64 numpy, so that the timed numbers rest on checked
# results.  (The parity tests proper, against the oracle, are under tests/.)
# A mismatch raises; nothing here runs inside a timed region.
# --------------------------------------------------------------------------- #


def _check(name: str, got, want, rtol: float, floor: float = 1e-30) -> None:
    """|got - want| <= rtol * (|want| + max(largest |want|, floor)), elementwise."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    bound = rtol * (np.abs(want) + max(float(np.abs(want).max()), floor))
    bad = ~(np.abs(got - want) <= bound)  # NaN counts as bad
    if bad.any():
        k = int(np.argmax(np.abs(got - want) / bound))
        raise RuntimeError(f"bench.py sanity check failed: {name}: got {got.flat[k]!r}, want {want.flat[k]!r} "
                           f"(rtol {rtol}, {int(bad.sum())} of {bad.size} values off)")


def _rows_to_host(dev, buf, rows, cols: int, np_dtype=np.float32) -> np.ndarray:
    """Rows `rows` of a contiguous fp32 (rows, cols) device buffer, one small copy per row."""
    out = np.empty((len(rows), cols), np_dtype)
    for i, r in enumerate(rows):
        dev.lib.mg_copy_to_host(out[i].ctypes.data_as(C.c_void_p), C.c_void_p(buf.data_ptr().value + r * cols * out.itemsize),
                                cols * out.itemsize, dev.stream)
    dev.synchronize()
    return out


def _verify_attention(q, k, v, do, o, lse, dq, dk, dv, B, H, S, D, causal: bool, rtol: float = 3e-2) -> None:
    """O, lse, dQ for sampled queries and dK, dV for sampled keys of two (batch, head) pairs.  Q, K, V and
    their gradients are (B, S, H, D); O and dO (B, H, S, D); lse (B, H, S).  (A causal query that sees one
    key has dQ = 0 exactly and the kernels leave the rounding of dP - delta: hence the absolute floor.)"""
    sc = 1.0 / np.sqrt(D)
    for (b, h) in ((0, 0), (B - 1, H - 1)):
        Q, K, V = (t[b, :, h, :].astype(np.float64) for t in (q, k, v))
        Oh, dO, L = o[b, h].astype(np.float64), do[b, h].astype(np.float64), lse[b, h].astype(np.float64)
        for i in (0, S // 2 + 1, S - 1):
            s = sc * (K @ Q[i])
            if causal:
                s[i + 1:] = -np.inf
            m = s.max()
            p = np.exp(s - m)
            l_ref = m + np.log(p.sum())
            p /= p.sum()
            _check(f"attention O[{b},{h},{i}]", Oh[i], p @ V, rtol)
            _check(f"attention lse[{b},{h},{i}]", [L[i]], [l_ref], 1e-3)
            ds = p * (V @ dO[i] - dO[i] @ Oh[i])
            _check(f"attention dQ[{b},{i},{h}]", dq[b, i, h], sc * (ds @ K), rtol, 1e-2)
        delta = np.einsum("sd,sd->s", dO, Oh)
        for j in (0, S // 2 - 1, S - 1):
            pj = np.exp(sc * (Q @ K[j]) - L)
            if causal:
                pj[:j] = 0.0
            _check(f"attention dV[{b},{j},{h}]", dv[b, j, h], pj @ dO, rtol, 1e-2)
            _check(f"attention dK[{b},{j},{h}]", dk[b, j, h], sc * ((pj * (dO @ V[j] - delta)) @ Q), rtol, 1e-2)


def bench_mlp(args, dev) -> dict:
    """README MLP, fp32: x (2048,4096) -> Linear 4096->4096 +ReLU -> LayerNorm(4096) -> Linear 4096->4096 +ReLU
    -> Linear 4096->10, cross-entropy on labels in [0,10).  Forward and backward through the C ABI."""
    from mograd_amd import F32, I32, AnyBuffer

    lib, st = dev.lib, dev.stream
    M, D, NC = 2048, 4096, 10
    bound = float(np.sqrt(6.0 / D))
    up = lambda a: AnyBuffer.from_numpy(dev, a)  # noqa: E731
    new = lambda n: AnyBuffer.create(F32, dev, n)  # noqa: E731
    x = up(_rng(3, 0).standard_normal((M, D), dtype=np.float32))
    w1, w2 = (up(_rng(3, i).uniform(-bound, bound, (D, D)).astype(np.float32)) for i in (1, 3))
    b1, b2 = (up(_rng(3, i).uniform(-bound, bound, D).astype(np.float32)) for i in (2, 4))
    w3 = up(_rng(3, 5).uniform(-bound, bound, (NC, D)).astype(np.float32))
    b3 = up(_rng(3, 6).uniform(-bound, bound, NC).astype(np.float32))
    gamma, beta = up(np.ones(D, np.float32)), up(np.zeros(D, np.float32))
    ids = AnyBuffer.from_numpy(dev, _rng(3, 7).integers(0, NC, M).astype(np.int32), I32)
    h1p, h1, ln, h2p, h2, logits = new(M * D), new(M * D), new(M * D), new(M * D), new(M * D), new(M * NC)
    loss, dlogits = new(1), new(M * NC)
    dh2, dh2p, dln, dh1, dh1p = new(M * D), new(M * D), new(M * D), new(M * D), new(M * D)
    dw1, dw2, dw3, db1, db2, db3, dg, dbt = new(D * D), new(D * D), new(NC * D), new(D), new(D), new(NC), new(D), new(D)
    P = lambda b: b.data_ptr()  # noqa: E731

    def linear(a, w, b, y, n_out, k):
        lib.mg_matmul_bias_bt(P(a), P(w), P(b), P(y), 1, M, n_out, k, k, 1, k, 1, M * k, n_out * k, F32, st)

    def fwd(i):
        linear(x, w1, b1, h1p, D, D)
        lib.mg_relu_grad(P(h1p), P(h1p), P(h1), M * D, F32, st)  # relu(v) == relu_grad(v, v)
        lib.mg_layer_norm_fwd(P(h1), P(gamma), P(beta), P(ln), M, D, 1e-5, F32, st)
        linear(ln, w2, b2, h2p, D, D)
        lib.mg_relu_grad(P(h2p), P(h2p), P(h2), M * D, F32, st)
        linear(h2, w3, b3, logits, NC, D)

    def bwd(i):
        lib.mg_cross_entropy_fused_ids(P(logits), P(ids), None, P(loss), P(dlogits), M, NC, F32, I32, st)
        lib.mg_linear_bwd(P(dlogits), P(h2), P(w3), P(dh2), P(dw3), P(db3), M, NC, D, F32, st)
        lib.mg_relu_grad(P(h2), P(dh2), P(dh2p), M * D, F32, st)
        lib.mg_linear_bwd(P(dh2p), P(ln), P(w2), P(dln), P(dw2), P(db2), M, D, D, F32, st)
        lib.mg_layer_norm_bwd(P(dln), P(h1), P(gamma), P(dh1), P(dg), P(dbt), M, D, 1e-5, F32, st)
        lib.mg_relu_grad(P(h1), P(dh1), P(dh1p), M * D, F32, st)
        lib.mg_linear_bwd(P(dh1p), P(x), P(w1), None, P(dw1), P(db1), M, D, D, F32, st)

    def step(i):
        fwd(i)
        bwd(i)

    # sampled rows of the second 4096 x 4096 layer's three products, and its db
    step(0)
    rows = [0, M // 3, M - 1]
    w2_h, b2_h = w2.to_numpy((D, D)).astype(np.float64), b2.to_numpy().astype(np.float64)
    ln_h, dy_h = ln.to_numpy((M, D)).astype(np.float64), dh2p.to_numpy((M, D)).astype(np.float64)
    _check("mlp Y = X W^T + b", _rows_to_host(dev, h2p, rows, D), ln_h[rows] @ w2_h.T + b2_h, 1e-4)
    _check("mlp dX = dY W", _rows_to_host(dev, dln, rows, D), dy_h[rows] @ w2_h, 1e-4)
    _check("mlp dW = dY^T X", _rows_to_host(dev, dw2, rows, D), dy_h[:, rows].T @ ln_h, 1e-4)
    _check("mlp db", db2.to_numpy(), dy_h.sum(axis=0), 1e-4)
    del w2_h, ln_h, dy_h

    ms = _time_steps(dev, step, args.warmup, args.steps)
    fl = 2.0 * M * D * D
    entries = [
        ("dX = dY W (mg_linear_bwd dx only, 2048x4096x4096)",
         lambda i: lib.mg_linear_bwd(P(dh2p), P(ln), P(w2), P(dln), None, None, M, D, D, F32, st), fl, "F", MFMA_F32_PEAK_TFLOPS),
        ("dW = dY^T X (mg_linear_bwd dw only)",
         lambda i: lib.mg_linear_bwd(P(dh2p), P(ln), P(w2), None, P(dw2), None, M, D, D, F32, st), fl, "F", MFMA_F32_PEAK_TFLOPS),
        ("db = sum rows dY (mg_sum_axis)",
         lambda i: lib.mg_sum_axis(P(dh2p), P(db2), 1, M, D, F32, st), M * D * 4 + D * 4, "B", None),
        ("Y = X W^T + b (mg_matmul_bias_bt)", lambda i: linear(ln, w2, b2, h2p, D, D), fl, "F", MFMA_F32_PEAK_TFLOPS),
    ]
    kernels = _kernel_table(dev, entries, max(10, min(args.steps, 50)))
    dom = min(kernels[:2], key=lambda r: r["frac_of_mfma_peak"])
    result = {
        "metric": "fwd+bwd step ms; per-bwd-kernel HBM GB/s or MFMA % of MI355X peak", "value": round(ms, 4),
        "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "README MLP fwd+bwd fp32: x (2048,4096) -> Linear 4096 +ReLU -> LayerNorm -> Linear 4096 "
                               "+ReLU -> Linear 10, cross-entropy, labels in [0,10)"},
        "roofline": {"bound": "mfma", "kernel": "gemm_f32_pipe_kernel, " + dom["name"], "achieved": dom["achieved_TFLOPs"],
                     "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": dom["frac_of_mfma_peak"],
                     "traffic": _measured_traffic("gemm_f32_pipe_kernel_mlp_step")},
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        # Linear gradients of one 4096x4096 layer on a slab of 128 of the 2048 rows (dX scales
        # with rows; dW's reduction length scales with rows), scaled x16; three layers' worth
        # is dominated by the two square ones.
        orc = _orc()
        cores = int(orc.orc_num_threads())
        rows = 128
        p = lambda a: a.ctypes.data_as(C.c_void_p)  # noqa: E731
        L = C.c_int64
        dy = _rng(3, 20).standard_normal((rows, D), dtype=np.float32)
        xs = _rng(3, 21).standard_normal((rows, D), dtype=np.float32)
        w = _rng(3, 22).uniform(-bound, bound, (D, D)).astype(np.float32)
        dxh, dwh, dbh = np.empty((rows, D), np.float32), np.empty((D, D), np.float32), np.empty(D, np.float32)

        def slab():
            orc.orc_linear_grad_x_f32(p(dy), p(w), p(dxh), L(rows), L(D), L(D))
            orc.orc_linear_grad_w_f32(p(dy), p(xs), p(dwh), L(rows), L(D), L(D))
            orc.orc_linear_grad_b_f32(p(dy), p(dbh), L(rows), L(D))

        slab_ms = _best_ms(slab)
        result["cpu_baseline"] = {
            "value": round(slab_ms * (M / rows), 1), "unit": "ms", "cores": cores, "kind": "port",
            "sample": f"dX + dW + db of one 4096x4096 Linear on {rows} of {M} rows ({slab_ms:.1f} ms) scaled x{M // rows}; "
                      f"one layer, not the whole step; best of 3 after a warm-up; OpenMP on {cores} threads"}
        result["c1_cpu"] = _c1_cpu_step(orc, cores)
    return result


def _c1_cpu_step(orc, cores: int) -> dict:
    """Configuration 1, which the reference itself could run on a CPU: MNIST-shaped MLP, fp32 input batch 64 x 784,
    Linear 784 -> 256 + ReLU, Linear 256 -> 10, softmax cross-entropy on class ids; one forward + backward step of the C
    restatement on this host (no GPU work)."""
    M, D0, D1, NC = 64, 784, 256, 10
    p = lambda a: a.ctypes.data_as(C.c_void_p)  # noqa: E731
    L = C.c_int64
    lin = lambda o, i, k: _rng(1, k).uniform(-np.sqrt(6.0 / i), np.sqrt(6.0 / i), (o, i)).astype(np.float32)  # noqa: E731
    x = _rng(1, 0).standard_normal((M, D0), dtype=np.float32)
    w1, w2 = lin(D1, D0, 1), lin(NC, D1, 3)
    b1, b2 = lin(1, D1, 2).reshape(-1), lin(1, NC, 4).reshape(-1)
    ids = _rng(1, 5).integers(0, NC, M).astype(np.int32)
    e = lambda *shape: np.empty(shape, np.float32)  # noqa: E731
    h, logits, dlogits, dh, dhp = e(M, D1), e(M, NC), e(M, NC), e(M, D1), e(M, D1)
    dw1, dw2, db1, db2 = e(D1, D0), e(NC, D1), e(D1), e(NC)
    up = np.ones(1, np.float32)
    orc.orc_cross_entropy_ids_f32.restype = C.c_float

    def step():
        orc.orc_matmul_bias_bt_f32(p(x), p(w1), p(b1), p(h), L(M), L(D1), L(D0))
        np.maximum(h, 0, out=h)
        orc.orc_matmul_bias_bt_f32(p(h), p(w2), p(b2), p(logits), L(M), L(NC), L(D1))
        orc.orc_cross_entropy_ids_f32(p(logits), p(ids), L(M), L(NC))
        orc.orc_cross_entropy_grad_ids_f32(p(logits), p(ids), p(up), p(dlogits), L(M), L(NC))
        orc.orc_linear_grad_x_f32(p(dlogits), p(w2), p(dh), L(M), L(NC), L(D1))
        orc.orc_linear_grad_w_f32(p(dlogits), p(h), p(dw2), L(M), L(NC), L(D1))
        orc.orc_linear_grad_b_f32(p(dlogits), p(db2), L(M), L(NC))
        orc.orc_relu_grad_f32(p(h), p(dh), p(dhp), L(M * D1))
        orc.orc_linear_grad_w_f32(p(dhp), p(x), p(dw1), L(M), L(D1), L(D0))
        orc.orc_linear_grad_b_f32(p(dhp), p(db1), L(M), L(D1))

    ms = _best_ms(step, 20)
    return {"value": round(ms, 4), "unit": "ms", "cores": cores, "kind": "port",
            "sample": "MNIST-shaped MLP (64 x 784 -> 256 + ReLU -> 10, cross-entropy on class ids), one whole forward + "
                      f"backward step in fp32 on the host, best of 20 after a warm-up; OpenMP on {cores} threads"}


def bench_attention(args, dev) -> dict:
    """Flash attention fwd+bwd, bf16 with fp32 accumulation: causal B8 H12 S1024 D64 (the step), and
    non-causal B2 H12 S4096 D64 in the kernel table."""
    from mograd_amd import BF16, F32, AnyBuffer

    lib, st = dev.lib, dev.stream

    def make(B, H, S, D, cfg, dtype=BF16):
        n = B * S * H * D
        q, k, v, do = (AnyBuffer.from_numpy(dev, _rng(4, cfg * 10 + i).standard_normal(n, dtype=np.float32), dtype)
                       for i in range(4))
        o, dq, dk, dv = (AnyBuffer.create(dtype, dev, n) for _ in range(4))
        lse = AnyBuffer.create(F32, dev, B * H * S)
        return q, k, v, do, o, dq, dk, dv, lse

    def runner(B, H, S, D, causal, bufs, dtype=BF16):
        q, k, v, do, o, dq, dk, dv, lse = bufs
        sc = 1.0 / float(np.sqrt(D))
        P = lambda b: b.data_ptr()  # noqa: E731
        f = lambda i: lib.mg_flash_attn_fwd(P(q), P(k), P(v), None, P(o), P(lse), B, S, H, D, sc, causal, 0, dtype, st)  # noqa: E731
        b = lambda i: lib.mg_flash_attn_bwd(P(do), P(o), P(q), P(k), P(v), None, P(lse), P(dq), P(dk), P(dv), B, S, H, D,  # noqa: E731
                                            sc, causal, 0, dtype, st)
        return f, b

    c1 = (8, 12, 1024, 64)
    c2 = (2, 12, 4096, 64)
    bufs1, bufs2, bufs3 = make(*c1, 1), make(*c2, 2), make(*c2, 3, F32)
    f1, b1 = runner(*c1, 1, bufs1)
    f2, b2 = runner(*c2, 0, bufs2)
    f3, b3 = runner(*c2, 0, bufs3, F32)  # the same tensors' shape in fp32: the fp32 matrix-core kernels
    for (Bc, Hc, Sc, Dc), causal, bufs, f, b, rtol in ((c1, True, bufs1, f1, b1, 3e-2), (c2, False, bufs2, f2, b2, 3e-2),
                                                       (c2, False, bufs3, f3, b3, 1e-4)):
        f(0)
        b(0)
        q_, k_, v_, do_, o_, dq_, dk_, dv_, lse_ = bufs
        bshd, bhsd = (Bc, Sc, Hc, Dc), (Bc, Hc, Sc, Dc)
        _verify_attention(q_.to_numpy(bshd), k_.to_numpy(bshd), v_.to_numpy(bshd), do_.to_numpy(bhsd), o_.to_numpy(bhsd),
                          lse_.to_numpy((Bc, Hc, Sc)), dq_.to_numpy(bshd), dk_.to_numpy(bshd), dv_.to_numpy(bshd),
                          Bc, Hc, Sc, Dc, causal, rtol)

    def step(i):
        f1(i)
        b1(i)

    ms = _time_steps(dev, step, args.warmup, args.steps)
    B, H, S, D = c1
    fl1 = B * H * S * S * D
    B2, H2, S2, D2 = c2
    fl2 = B2 * H2 * S2 * S2 * D2
    entries = [
        ("flash_attn_bwd bf16 causal B8 H12 S1024 D64 (5 B H S^2 D)", b1, 5.0 * fl1, "F", MFMA_BF16_PEAK_TFLOPS),
        ("flash_attn_fwd bf16 causal B8 H12 S1024 D64 (2 B H S^2 D)", f1, 2.0 * fl1, "F", MFMA_BF16_PEAK_TFLOPS),
        ("flash_attn_bwd bf16 B2 H12 S4096 D64 (10 B H S^2 D)", b2, 10.0 * fl2, "F", MFMA_BF16_PEAK_TFLOPS),
        ("flash_attn_fwd bf16 B2 H12 S4096 D64 (4 B H S^2 D)", f2, 4.0 * fl2, "F", MFMA_BF16_PEAK_TFLOPS),
        ("flash_attn_bwd fp32 B2 H12 S4096 D64 (10 B H S^2 D; not a BASELINE configuration: fp32 tensors on the fp32 "
         "matrix pipe)", b3, 10.0 * fl2, "F", MFMA_F32_PEAK_TFLOPS),
        ("flash_attn_fwd fp32 B2 H12 S4096 D64 (4 B H S^2 D; likewise)", f3, 4.0 * fl2, "F", MFMA_F32_PEAK_TFLOPS),
    ]
    kernels = _kernel_table(dev, entries, max(10, min(args.steps, 50)))
    dom = kernels[0]
    result = {
        "metric": "fwd+bwd step ms; per-bwd-kernel HBM GB/s or MFMA % of MI355X peak", "value": round(ms, 4),
        "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "causal flash-attention fwd+bwd bf16 (fp32 accumulate) B8 H12 S1024 D64, scale 1/8; "
                               "kernel table also has non-causal B2 H12 S4096 D64"},
        "roofline": {"bound": "mfma", "kernel": "attn_bwd_mfma_kernel (dK/dV and dQ walks) + attn_delta_rows_kernel "
                                                "(mg_flash_attn_bwd, causal S1024)",
                     "achieved": dom["achieved_TFLOPs"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": dom["frac_of_mfma_peak"], "traffic": _measured_traffic("attn_bwd_mfma_kernel_b8h12s1024")},
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        # fp32 naive O(S^2) attention (the reference's oracle structure) on 4 of the 96 (b,h)
        # pairs of the causal configuration, scaled x24.
        orc = _orc()
        cores = int(orc.orc_num_threads())
        p = lambda a: a.ctypes.data_as(C.c_void_p)  # noqa: E731
        L = C.c_int64
        Bs, Hs = 1, 4
        n = Bs * S * Hs * D
        q, k, v, do = (_rng(4, 50 + i).standard_normal(n, dtype=np.float32) for i in range(4))
        o, dq, dk, dv = (np.empty(n, np.float32) for _ in range(4))
        lse = np.empty(Bs * Hs * S, np.float32)

        def slab():
            orc.orc_sdpa_fwd_f32(p(q), p(k), p(v), None, 0, 1, p(o), p(lse), L(Bs), L(S), L(Hs), L(D), C.c_float(0.125),
                                 L(Bs * Hs))
            orc.orc_sdpa_bwd_f32(p(q), p(k), p(v), p(do), None, 0, 1, p(dq), p(dk), p(dv), L(Bs), L(S), L(Hs), L(D),
                                 C.c_float(0.125), L(Bs * Hs))

        slab_ms = _best_ms(slab)
        scale_up = (B * H) // (Bs * Hs)
        result["cpu_baseline"] = {
            "value": round(slab_ms * scale_up, 1), "unit": "ms", "cores": cores, "kind": "port",
            "sample": f"naive fp32 attention fwd+bwd on {Bs * Hs} of {B * H} (batch, head) pairs of the causal "
                      f"configuration ({slab_ms:.1f} ms) scaled x{scale_up}; best of 3 after a warm-up; OpenMP on {cores} threads"}
    return result


def bench_gpt(args, dev) -> dict:
    """Character-level GPT training step (examples/tinyshakespear/model.mojo shape): vocab 65, context 256,
    batch 64, 6 layers, d_model 384, 6 heads, MLP 4x, pre-LayerNorm, bf16 activations with fp32 master weights,
    token ids uniform in [0, 65); forward, loss and every parameter gradient."""
    from mograd_amd import BF16, F32, I32, AnyBuffer
    from mograd_amd.tiny_transformer import TinyTransformer, init_params

    lib, st = dev.lib, dev.stream
    V, d, ff, L, H, B, T = 65, 384, 1536, 6, 6, 64, 256
    n, dh = B * T, d // H
    model = TinyTransformer(dev, V, d, ff, L, H, compute_dtype=BF16)
    model.load_params(init_params(_rng(5, 0), V, d, ff, L))
    ids = AnyBuffer.from_numpy(dev, _rng(5, 1).integers(0, V, (B, T)).astype(np.int32))
    labels = AnyBuffer.from_numpy(dev, _rng(5, 2).integers(0, V, (B, T)).astype(np.int32))

    # the end of the chain on this step's own tensors: the loss from the logits, sampled rows of
    # dlogits, the 65-symbol head's weight gradient from dlogits and the last hidden state, and
    # every gradient finite
    model.step(ids, labels, B, T)
    lg = model.tmp["logits"].to_numpy((n, V)).astype(np.float64)
    lab = labels.to_numpy().reshape(-1)
    lsm = lg - lg.max(axis=1, keepdims=True)
    lsm -= np.log(np.exp(lsm).sum(axis=1, keepdims=True))
    _check("gpt loss", [model.loss.item()], [-lsm[np.arange(n), lab].mean()], 2e-3)
    dl = model.tmp["dlogits"].to_numpy((n, V)).astype(np.float64)
    rows = [0, n // 2 + 5, n - 1]
    want = np.exp(lsm[rows])
    for n_, r in enumerate(rows):
        want[n_, lab[r]] -= 1.0
    _check("gpt dlogits", dl[rows], want / n, 1e-2)
    grads = model.gradients()
    _check("gpt d lm_head", grads["lm_head"], dl.T @ model.h[L].to_numpy((n, d)).astype(np.float64), 2e-2)
    if not np.all(np.isfinite(model.grads.to_numpy())):
        raise RuntimeError("bench.py sanity check failed: gpt gradients are not all finite")
    del lg, lsm, dl, grads

    ms = _time_steps(dev, lambda i: model.step(ids, labels, B, T), args.warmup, args.steps)
    loss = model.loss.item()

    # forward / backward split, from events recorded on the library's stream inside the step
    iters = max(5, min(args.steps, 20))
    ev = [[C.c_void_p() for _ in range(3)] for _ in range(iters)]
    for row in ev:
        for e in row:
            lib.mg_event_create(C.byref(e))
    for row in ev:
        lib.mg_event_record(row[0], st)
        model.step(ids, labels, B, T, marks=lambda which, row=row: lib.mg_event_record(row[1 if which == "forward" else 2], st))
    dev.synchronize()
    fwd_ms, bwd_ms = [], []
    for row in ev:
        a, b = C.c_float(), C.c_float()
        lib.mg_event_elapsed_ms(row[0], row[1], C.byref(a))
        lib.mg_event_elapsed_ms(row[1], row[2], C.byref(b))
        fwd_ms.append(a.value)
        bwd_ms.append(b.value)
        for e in row:
            lib.mg_event_destroy(e)

    # per-kernel table at the step's shapes
    P = lambda b: b.data_ptr()  # noqa: E731
    new = lambda numel, dt=BF16: AnyBuffer.create(dt, dev, numel)  # noqa: E731
    rnd = lambda numel, k: AnyBuffer.from_numpy(dev, _rng(5, 10 + k).standard_normal(numel, dtype=np.float32), BF16)  # noqa: E731
    x_d, x_ff, dy_d, dy_ff = rnd(n * d, 0), rnd(n * ff, 1), rnd(n * d, 2), rnd(n * ff, 3)
    w_dd, w_fd, w_df, w_vd = rnd(d * d, 4), rnd(ff * d, 5), rnd(d * ff, 6), rnd(V * d, 7)
    bias_f, gam, bet = rnd(ff, 8), rnd(d, 9), rnd(d, 10)
    out_d, out_ff, out_v, dlog = new(n * d), new(n * ff), new(n * V), new(n * V)
    dw_big, db_big, dgam, dbet = new(ff * d), new(ff), new(d), new(d)
    big_ids = AnyBuffer.from_numpy(dev, _rng(5, 9).integers(0, 50304, 8192).astype(np.int32), I32)
    big_table = new(50304 * 768)
    mean, rstd, lse, loss1 = new(n, F32), new(n, F32), new(B * H * T, F32), new(1)
    qkv, o, do, dqkv = rnd(3 * n * d, 11), new(n * d), rnd(n * d, 14), rnd(3 * n * d, 15)  # Q | K | V per token
    w_qkv = rnd(3 * d * d, 12)  # the stacked (3d, d) projection weight
    i64 = lambda *a: (C.c_int64 * len(a))(*a)  # noqa: E731
    sc = 1.0 / float(np.sqrt(dh))
    lib.mg_layer_norm_fwd_stats(P(x_d), P(gam), P(bet), P(out_d), P(mean), P(rstd), n, d, 1e-5, BF16, st)
    lib.mg_flash_attn_fwd_packed(P(qkv), None, P(o), P(lse), B, T, H, dh, sc, 1, 0, BF16, st)
    lib.mg_matmul_bt(P(x_d), P(w_vd), P(out_v), 1, n, V, d, d, 1, d, 1, n * d, V * d, BF16, st)

    def mm(x, w, out, N, K, bias=None):
        if bias is None:
            return lambda i: lib.mg_matmul_bt(P(x), P(w), P(out), 1, n, N, K, K, 1, K, 1, n * K, N * K, BF16, st)
        return lambda i: lib.mg_matmul_bias_bt(P(x), P(w), P(bias), P(out), 1, n, N, K, K, 1, K, 1, n * K, N * K, BF16, st)

    # The step's form of the Linear backward: dW and db are fp32 sums whose second stage is left
    # on a list (mg_linear_bwd_deferred) and run by one launch per step (mg_finish_deferred, timed
    # below as a row of its own).  Every timed call gets fresh partial-result blocks, as in the step.
    pending = C.c_void_p()
    lib.mg_deferred_create(C.byref(pending))
    dw32, db32, dg32, dbt32 = new(ff * d, F32), new(ff, F32), new(d, F32), new(d, F32)

    def lbwd(dy, x, w, dx, N, K, db=None):
        return lambda i: lib.mg_linear_bwd_deferred(P(dy), P(x), P(w), P(dx), P(dw32), P(db32) if db else None, n, N, K, 0, 0,
                                                    BF16, F32, pending, st)

    PF = MFMA_BF16_PEAK_TFLOPS
    e2 = 2  # bytes per bf16
    # These rows call a kernel again and again on the same 25-150 MB of operands, which then sit in
    # the 256 MB memory-side cache, as they do inside the step (each kernel reads what the previous
    # one wrote): their rates describe the step, not an HBM stream, and exceed what this device
    # streams from cold HBM (0.65-0.77 of the nominal peak, see the ln_ce calibration rows).
    CACHED = "operands resident in the 256 MB memory-side cache, a cache rate, not an HBM stream"
    attn_fl = B * H * T * T * dh
    entries = [
        ("linear_bwd_deferred dX+dW bf16, stacked Q|K|V projection (16384, 1152<-384)", lbwd(dqkv, x_d, w_qkv, out_d, 3 * d, d),
         12.0 * n * d * d, "F", PF),
        ("linear_bwd_deferred dX+dW bf16 (16384, 384<-384)", lbwd(dy_d, x_d, w_dd, out_d, d, d), 4.0 * n * d * d, "F", PF),
        ("linear_bwd_deferred dX+dW+db bf16 (16384, 1536<-384)", lbwd(dy_ff, x_d, w_fd, out_d, ff, d, db_big), 4.0 * n * d * ff, "F", PF),
        ("linear_bwd_deferred dX+dW bf16 (16384, 384<-1536)", lbwd(dy_d, x_ff, w_df, out_ff, d, ff), 4.0 * n * d * ff, "F", PF),
        ("linear_bwd_deferred dX+dW bf16 lm_head (16384, 65<-384)", lbwd(dlog, x_d, w_vd, out_d, V, d), 4.0 * n * d * V, "F", PF),
        ("matmul_bt bf16, stacked Q|K|V projection (16384, 1152<-384)", mm(x_d, w_qkv, dqkv, 3 * d, d), 6.0 * n * d * d, "F", PF),
        ("matmul_bt bf16 (16384, 384<-384)", mm(x_d, w_dd, out_d, d, d), 2.0 * n * d * d, "F", PF),
        ("matmul_bias_bt bf16 (16384, 1536<-384)", mm(x_d, w_fd, out_ff, ff, d, bias_f), 2.0 * n * d * ff, "F", PF),
        ("matmul_bt bf16 (16384, 384<-1536)", mm(x_ff, w_df, out_d, d, ff), 2.0 * n * d * ff, "F", PF),
        ("matmul_bt bf16 lm_head (16384, 65<-384)", mm(x_d, w_vd, out_v, V, d), 2.0 * n * d * V, "F", PF),
        ("flash_attn_bwd_packed bf16 causal B64 H6 S256 D64 (5 B H S^2 D)",
         lambda i: lib.mg_flash_attn_bwd_packed(P(do), P(o), P(qkv), None, P(lse), P(dqkv), B, T, H, dh, sc, 1, 0, BF16, st),
         5.0 * attn_fl, "F", PF),
        ("flash_attn_fwd_packed bf16 causal B64 H6 S256 D64 (2 B H S^2 D)",
         lambda i: lib.mg_flash_attn_fwd_packed(P(qkv), None, P(o), P(lse), B, T, H, dh, sc, 1, 0, BF16, st), 2.0 * attn_fl, "F", PF),
        ("layer_norm_bwd_stats_deferred bf16 (16384, 384), dx accumulated in place, dgamma/dbeta sums deferred (not in "
         "the step since the Linear backward after each LayerNorm carries it: the next two rows); " + CACHED,
         lambda i: lib.mg_layer_norm_bwd_stats_deferred(P(dy_d), P(x_d), P(gam), P(mean), P(rstd), P(out_d), P(out_d), P(dg32),
                                                        P(dbt32), n, d, BF16, F32, pending, st),
         4 * n * d * e2 + 2 * n * 4 + 3 * d * e2, "B", None),
        ("linear_bwd_layer_norm_bwd bf16, stacked Q|K|V projection (16384, 1152<-384): linear_bwd_deferred plus the "
         "backward of the LayerNorm that feeds the layer, from the dX tiles (4 M N K FLOP counted; in the step)",
         lambda i: lib.mg_linear_bwd_layer_norm_bwd(P(dqkv), P(x_d), P(w_qkv), P(x_ff), P(gam), P(mean), P(rstd), P(out_d),
                                                    P(dw32), None, P(dg32), P(dbt32), n, 3 * d, d, 1, BF16, F32, pending, st),
         12.0 * n * d * d, "F", PF),
        ("linear_bwd_layer_norm_bwd bf16 (16384, 1536<-384) with db: likewise (in the step)",
         lambda i: lib.mg_linear_bwd_layer_norm_bwd(P(dy_ff), P(x_d), P(w_fd), P(x_ff), P(gam), P(mean), P(rstd), P(out_d),
                                                    P(dw32), P(db32), P(dg32), P(dbt32), n, ff, d, 1, BF16, F32, pending, st),
         4.0 * n * d * ff, "F", PF),
        ("layer_norm_fwd_stats bf16 (16384, 384); " + CACHED,
         lambda i: lib.mg_layer_norm_fwd_stats(P(x_d), P(gam), P(bet), P(out_d), P(mean), P(rstd), n, d, 1e-5, BF16, st),
         2 * n * d * e2 + 2 * n * 4 + 2 * d * e2, "B", None),
        ("cross_entropy_fused_ids bf16 (16384, 65)",
         lambda i: lib.mg_cross_entropy_fused_ids(P(out_v), P(labels), None, P(loss1), P(dlog), n, V, BF16, I32, st),
         2 * n * V * e2 + n * 4 + e2, "B", None),
        ("add bf16 (16384 x 384) (not in the step since LayerNorm backward accumulates); " + CACHED, lambda i: lib.mg_add(P(x_d), P(dy_d), P(out_d), n * d, BF16, st), 3 * n * d * e2, "B", None),
        ("relu bf16 (16384 x 1536) (not in the step: the product's epilogue applies it); " + CACHED, lambda i: lib.mg_relu(P(x_ff), P(out_ff), n * ff, BF16, st), 2 * n * ff * e2, "B", None),
        ("relu_grad bf16 (16384 x 1536) (not in the step: the dX product's epilogue applies it); " + CACHED, lambda i: lib.mg_relu_grad(P(x_ff), P(dy_ff), P(out_ff), n * ff, BF16, st), 3 * n * ff * e2, "B", None),
        ("contiguous bf16 (B,H,T,dh) -> (B,T,H,dh) (not in the step since attention writes (B,T,H,dh)); " + CACHED,
         lambda i: lib.mg_contiguous(P(o), P(out_d), 4, i64(B, T, H, dh), i64(H * T * dh, dh, T * dh, 1), BF16, st), 2 * n * d * e2, "B", None),
        ("gather bf16 16384 rows of (65, 384)", lambda i: lib.mg_gather(P(w_vd), P(ids), P(out_d), n, V, d, d, 1, I32, BF16, st),
         n * d * e2 + n * 4, "B", None),
        ("scatter_add bf16 16384 rows into (65, 384)", lambda i: lib.mg_scatter_add(P(ids), P(dy_d), P(dw_big), n, V, d, I32, BF16, st),
         n * d * e2 + n * 4 + V * d * e2, "B", None),
        ("scatter_add bf16 8192 rows of 768 into a (50304, 768) table (not in the step: a GPT-2-sized embedding gradient, "
         "indices bucketed by row first)",
         lambda i: lib.mg_scatter_add(P(big_ids), P(x_ff), P(big_table), 8192, 50304, 768, I32, BF16, st),
         8192 * 768 * e2 + 8192 * 4 + 50304 * 768 * e2, "B", None),
        ("cast fp32 -> bf16 parameter arena; " + CACHED, lambda i: lib.mg_cast(P(model.master), P(model.work), model.total, F32, BF16, st),
         model.total * 6, "B", None),
    ]
    # A deferred call keeps its partial-result blocks until the list is finished, so every call of
    # a timed run takes fresh blocks from the pool: one untimed run of the same length first, so
    # that the pool holds them (as it does from the second training step on) and the timed calls
    # do not wait for the driver's allocator.
    table_iters = max(10, min(args.steps, 30))
    for name, fn, *_ in entries:
        if "_deferred" in name:
            for _ in range(table_iters + 1):
                fn(0)
            lib.mg_finish_deferred(pending, st)
    dev.synchronize()
    kernels = _kernel_table(dev, entries, table_iters)
    lib.mg_finish_deferred(pending, st)

    # The one launch that finishes a step's second-stage sums: the list is filled with what a step
    # leaves on it (4 Linear layers and 2 LayerNorms per block, the head, the embedding), then the
    # finishing launch alone is timed.
    def fill_pending():
        for _ in range(L):
            for f in (entries[0][1], entries[1][1], entries[2][1], entries[3][1]):
                f(0)
            for _ in range(2):
                lib.mg_layer_norm_bwd_stats_deferred(P(dy_d), P(x_d), P(gam), P(mean), P(rstd), P(out_d), P(out_d), P(dg32),
                                                     P(dbt32), n, d, BF16, F32, pending, st)
        entries[4][1](0)
        lib.mg_scatter_add_deferred(P(ids), P(dy_d), P(dw32), n, V, d, I32, BF16, F32, pending, st)

    fin_ms = []
    e0, e1 = C.c_void_p(), C.c_void_p()
    lib.mg_event_create(C.byref(e0))
    lib.mg_event_create(C.byref(e1))
    for _ in range(6):
        fill_pending()
        n_pending = int(lib.mg_deferred_pending(pending))
        lib.mg_event_record(e0, st)
        lib.mg_finish_deferred(pending, st)
        lib.mg_event_record(e1, st)
        t = C.c_float()
        lib.mg_event_elapsed_ms(e0, e1, C.byref(t))
        fin_ms.append(t.value)
    lib.mg_event_destroy(e0)
    lib.mg_event_destroy(e1)
    lib.mg_deferred_destroy(pending)
    fin = float(np.mean(fin_ms[1:]))
    kernels.insert(5, {"name": f"finish_deferred: the {n_pending} second-stage sums of a step (dW K ranges, db, dgamma/dbeta, "
                               "embedding slabs) in one launch, fp32 results", "mean_ms": round(fin, 5),
                       "median_ms": round(float(np.median(fin_ms[1:])), 5)})

    # The same step as the rule tables produce it: forward graph in plain ops, gradient() over
    # GRAD_RULES, Simplifier(GPU_REWRITES()), evaluate_many with deferred sums (bit-identical
    # results, tests/test_grad_rules.py).  The graph is rebuilt every step, as the reference's lazy
    # tensors do; `host_graph_ms` is the part of that spent building, differentiating and
    # rewriting the graph on the host, which overlaps the GPU only partly in this Python mirror.
    from mograd_amd.rewrites import GPU_REWRITES, Simplifier
    from mograd_amd.runtime import Layout, Node, gradient

    via_ms = _time_steps(dev, lambda i: model.step_via_rules(ids, labels, B, T), 2, max(5, min(args.steps, 20)))
    kept_ms = _time_steps(dev, lambda i: model.step_via_rules(ids, labels, B, T, reuse_graph=True), 2,
                          max(5, min(args.steps, 20)))

    def host_graph():
        loss_node, leaves = model.graph(ids, labels, B, T)
        grads = gradient(loss_node, Node.leaf(Layout(1), BF16), [v for k, v in leaves.items() if not k.endswith((".wk", ".wv"))])
        Simplifier(GPU_REWRITES()).run_many([loss_node] + grads)

    via_rules = {"ms_per_step_via_rules": round(via_ms, 4), "host_graph_ms": round(_best_ms(host_graph), 4),
                 "ms_per_step_via_rules_graph_kept": round(kept_ms, 4),
                 "note": "gradient() + Simplifier(GPU_REWRITES()) + evaluate_many(deferred sums) over the model's node graph, "
                         "rebuilt every step (graph_kept: built once, evaluated every step); same kernels and bits as the "
                         "hand-sequenced step, whose time is `value`; the difference is host time of this Python mirror "
                         "(one pool allocation and one ctypes call per node)"}
    flops = model.flops_per_step(B, T)
    tf = flops / (ms * 1e-3) / 1e12
    # The backward kernel that takes most of the step: linear_bwd_16bit_kernel (dX and dW of one
    # Linear layer in one launch), timed through mg_linear_bwd_deferred as the step calls it: the
    # sums of dW's K ranges are part of the step's one finishing launch (its own row).  Each of
    # the four layer shapes runs once per block.  `kernel_only_frac` is the same figure from the
    # kernel's average duration in the committed rocprofv3 trace of this workload.
    lin = kernels[:4]
    trace_us = _trace_kernel_us("linear_bwd_16bit_kernel_gpt_step")
    lin_flops = sum(k["algorithmic_flops"] for k in lin)
    lin_ms = sum(k["mean_ms"] for k in lin)
    lin_tf = lin_flops / (lin_ms * 1e-3) / 1e12
    result = {
        "metric": "fwd+bwd step ms; per-bwd-kernel HBM GB/s or MFMA % of MI355X peak", "value": round(ms, 4),
        "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "char-level GPT training step: vocab 65, ctx 256, batch 64, 6 layers, d_model 384, 6 heads, "
                               "MLP 4x, pre-LayerNorm, bf16 activations / fp32 master weights, ids uniform in [0,65); "
                               "forward + loss + all parameter gradients",
                   "tokens_per_step": n, "loss": round(loss, 4)},
        "phases_ms": {"forward": round(float(np.mean(fwd_ms)), 4), "backward": round(float(np.mean(bwd_ms)), 4)},
        "roofline": {"bound": "mfma",
                     "kernel": "linear_bwd_16bit_kernel: mg_linear_bwd_deferred at the block's four layer shapes, "
                               "4 M N K FLOP each, mean over the four",
                     "achieved": round(lin_tf, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(lin_tf / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": _measured_traffic("linear_bwd_16bit_kernel_gpt_step"),
                     "algorithmic_flops": lin_flops / 4, "launch_ms": round(lin_ms / 4, 5),
                     "kernel_only_frac": (round(lin_flops / 4 / (trace_us * 1e-6) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)
                                          if trace_us else None),
                     "share_of_step": round(L * lin_ms / ms, 3)},
        "whole_step": {"algorithmic_flops": flops, "achieved_TFLOPs": round(tf, 1),
                       "frac_of_mfma_peak": round(tf / MFMA_BF16_PEAK_TFLOPS, 4)},
        "via_rules": via_rules,
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = _gpt_cpu_baseline(V, d, ff, L, H, B, T)
    return result


def _gpt_cpu_baseline(V, d, ff, L, H, B, T):
    """fp32 C restatement of one transformer block (forward + backward) on 4 of the 64 sequences, scaled by
    16 x 6 layers; embedding, lm_head and the loss (under 2% of the work) are left out."""
    orc = _orc()
    cores = int(orc.orc_num_threads())
    p = lambda a: a.ctypes.data_as(C.c_void_p)  # noqa: E731
    Li, F = C.c_int64, C.c_float
    Bs = 4
    n, dh = Bs * T, d // H
    r = lambda k, *shape: _rng(5, 100 + k).standard_normal(shape, dtype=np.float32)  # noqa: E731
    x, dy = r(0, n, d), r(1, n, d)
    g, be = np.ones(d, np.float32), np.zeros(d, np.float32)
    w = {name: r(2 + i, *shape) * 0.05 for i, (name, shape) in enumerate(
        [("wq", (d, d)), ("wk", (d, d)), ("wv", (d, d)), ("wo", (d, d)), ("w1", (ff, d)), ("w2", (d, ff))])}
    b1 = np.zeros(ff, np.float32)
    e = lambda *shape: np.empty(shape, np.float32)  # noqa: E731
    x1, q, k, v, o, ctx, proj, hmid, x2, a, f = e(n, d), e(n, d), e(n, d), e(n, d), e(n, d), e(n, d), e(n, d), e(n, d), e(n, d), e(n, ff), e(n, d)
    lse = e(Bs * H * T)
    da, dxa, dxb, dxc, dres, dq, dk, dv, dctx = e(n, ff), e(n, d), e(n, d), e(n, d), e(n, d), e(n, d), e(n, d), e(n, d), e(n, d)
    dw_dd, dw_fd, dw_df, db1, dg, db = e(d, d), e(ff, d), e(d, ff), e(ff), e(d), e(d)

    def lin(xi, wi, bi, yi, N, K):
        orc.orc_matmul_bias_bt_f32(p(xi), p(wi), p(bi) if bi is not None else None, p(yi), Li(n), Li(N), Li(K))

    def lin_bwd(dyi, xi, wi, dxi, dwi, N, K, dbi=None):
        orc.orc_linear_grad_x_f32(p(dyi), p(wi), p(dxi), Li(n), Li(N), Li(K))
        orc.orc_linear_grad_w_f32(p(dyi), p(xi), p(dwi), Li(n), Li(N), Li(K))
        if dbi is not None:
            orc.orc_linear_grad_b_f32(p(dyi), p(dbi), Li(n), Li(N))

    def block():
        orc.orc_layer_norm_fwd_f32(p(x), p(g), p(be), p(x1), Li(n), Li(d), F(1e-5))
        lin(x1, w["wq"], None, q, d, d)
        lin(x1, w["wk"], None, k, d, d)
        lin(x1, w["wv"], None, v, d, d)
        orc.orc_sdpa_fwd_f32(p(q), p(k), p(v), None, 0, 1, p(o), p(lse), Li(Bs), Li(T), Li(H), Li(dh), F(0.125), Li(Bs * H))
        ctx[:] = o.reshape(Bs, H, T, dh).transpose(0, 2, 1, 3).reshape(n, d)
        lin(ctx, w["wo"], None, proj, d, d)
        np.add(x, proj, out=hmid)
        orc.orc_layer_norm_fwd_f32(p(hmid), p(g), p(be), p(x2), Li(n), Li(d), F(1e-5))
        lin(x2, w["w1"], b1, a, ff, d)
        np.maximum(a, 0, out=a)
        lin(a, w["w2"], None, f, d, ff)
        # backward
        lin_bwd(dy, a, w["w2"], da, dw_df, d, ff)
        orc.orc_relu_grad_f32(p(a), p(da), p(da), Li(n * ff))
        lin_bwd(da, x2, w["w1"], dxa, dw_fd, ff, d, db1)
        orc.orc_layer_norm_bwd_f32(p(dxa), p(hmid), p(g), p(dres), p(dg), p(db), Li(n), Li(d), F(1e-5), Li(256))
        lin_bwd(dres, ctx, w["wo"], dctx, dw_dd, d, d)
        do = np.ascontiguousarray(dctx.reshape(Bs, T, H, dh).transpose(0, 2, 1, 3))
        orc.orc_sdpa_bwd_f32(p(q), p(k), p(v), p(do), None, 0, 1, p(dq), p(dk), p(dv), Li(Bs), Li(T), Li(H), Li(dh), F(0.125), Li(Bs * H))
        lin_bwd(dq, x1, w["wq"], dxa, dw_dd, d, d)
        lin_bwd(dk, x1, w["wk"], dxb, dw_dd, d, d)
        lin_bwd(dv, x1, w["wv"], dxc, dw_dd, d, d)
        np.add(dxa, dxb, out=dxa)
        np.add(dxa, dxc, out=dxa)
        orc.orc_layer_norm_bwd_f32(p(dxa), p(x), p(g), p(dres), p(dg), p(db), Li(n), Li(d), F(1e-5), Li(256))

    one = _best_ms(block)
    scale_up = (B // Bs) * L
    return {"value": round(one * scale_up, 1), "unit": "ms", "cores": cores, "kind": "port",
            "sample": f"one transformer block fwd+bwd in fp32 on {Bs} of {B} sequences ({one:.1f} ms) scaled x{scale_up} "
                      f"(16 batch slices x {L} layers); embedding, lm_head and loss left out; best of 3 after a warm-up; OpenMP on {cores} threads"}


def bench_ln_ce(args, dev) -> dict:
    """LayerNorm fwd+bwd fp32 (2048,4096) plus fused softmax-cross-entropy fwd+bwd fp32 (8192,50304), int32 labels."""
    from mograd_amd import F32, I32, AnyBuffer

    lib = dev.lib
    st = dev.stream

    # ---- inputs, resident in HBM -------------------------------------------------------
    # LayerNorm: four rotating sets (4 x 100 MB) so that no set is still in the 256 MB
    # memory-side cache when it is used again.
    LN_SETS = 4
    gamma = AnyBuffer.from_numpy(dev, _rng(2, 1).uniform(0.5, 1.5, LN_COLS).astype(np.float32))
    beta = AnyBuffer.from_numpy(dev, (_rng(2, 2).standard_normal(LN_COLS) * 0.1).astype(np.float32))
    ln_sets = []
    for s in range(LN_SETS):
        x = AnyBuffer.from_numpy(dev, _rng(2, 100 + s).standard_normal((LN_ROWS, LN_COLS), dtype=np.float32))
        dy = AnyBuffer.from_numpy(dev, _rng(2, 200 + s).standard_normal((LN_ROWS, LN_COLS), dtype=np.float32))
        y = AnyBuffer.create(F32, dev, LN_ROWS * LN_COLS)
        dx = AnyBuffer.create(F32, dev, LN_ROWS * LN_COLS)
        ln_sets.append((x, dy, y, dx))
    dgamma = AnyBuffer.create(F32, dev, LN_COLS)
    dbeta = AnyBuffer.create(F32, dev, LN_COLS)

    # Cross-entropy: 1.65 GB of logits, uploaded in slabs.
    logits = AnyBuffer.create(F32, dev, CE_ROWS * CE_COLS)
    dlogits = AnyBuffer.create(F32, dev, CE_ROWS * CE_COLS)
    rng = _rng(2, 10)
    slab = 1024
    for r0 in range(0, CE_ROWS, slab):
        part = rng.standard_normal((slab, CE_COLS), dtype=np.float32) * 2.0
        lib.mg_copy_to_device(C.c_void_p(logits.data_ptr().value + r0 * CE_COLS * 4), part.ctypes.data_as(C.c_void_p),
                              part.nbytes, st)
    ids = AnyBuffer.from_numpy(dev, _rng(2, 11).integers(0, CE_COLS, CE_ROWS).astype(np.int32), I32)
    loss = AnyBuffer.create(F32, dev, 1)

    def ln_fwd(i):
        x, dy, y, dx = ln_sets[i % LN_SETS]
        lib.mg_layer_norm_fwd(x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), y.data_ptr(), LN_ROWS, LN_COLS, 1e-5,
                              F32, st)

    def ln_bwd(i):
        x, dy, y, dx = ln_sets[i % LN_SETS]
        lib.mg_layer_norm_bwd(dy.data_ptr(), x.data_ptr(), gamma.data_ptr(), dx.data_ptr(), dgamma.data_ptr(),
                              dbeta.data_ptr(), LN_ROWS, LN_COLS, 1e-5, F32, st)

    def ce_fused(i):
        lib.mg_cross_entropy_fused_ids(logits.data_ptr(), ids.data_ptr(), None, loss.data_ptr(), dlogits.data_ptr(),
                                       CE_ROWS, CE_COLS, F32, I32, st)

    def step(i):
        ln_fwd(i)
        ln_bwd(i)
        ce_fused(i)

    # sampled rows of the cross-entropy gradient and of the LayerNorm outputs
    step(0)
    rows = [0, CE_ROWS // 2 + 3, CE_ROWS - 1]
    lg = _rows_to_host(dev, logits, rows, CE_COLS).astype(np.float64)
    idh = ids.to_numpy()
    pr = np.exp(lg - lg.max(axis=1, keepdims=True))
    pr /= pr.sum(axis=1, keepdims=True)
    for n_, r in enumerate(rows):
        pr[n_, idh[r]] -= 1.0
    _check("cross-entropy dlogits", _rows_to_host(dev, dlogits, rows, CE_COLS), pr / CE_ROWS, 1e-4)
    if not np.isfinite(loss.item()) or loss.item() <= 0.0:
        raise RuntimeError(f"bench.py sanity check failed: cross-entropy loss {loss.item()!r}")
    x0, dy0, y0, dx0 = ln_sets[0]
    lrows = [0, LN_ROWS // 2, LN_ROWS - 1]
    xh, dyh = (_rows_to_host(dev, t, lrows, LN_COLS).astype(np.float64) for t in (x0, dy0))
    gh, bh_ = gamma.to_numpy().astype(np.float64), beta.to_numpy().astype(np.float64)
    mu, var = xh.mean(axis=1, keepdims=True), xh.var(axis=1, keepdims=True)
    xhat = (xh - mu) / np.sqrt(var + 1e-5)
    _check("layer_norm y", _rows_to_host(dev, y0, lrows, LN_COLS), xhat * gh + bh_, 1e-4)
    dyg = dyh * gh
    dx_ref = (dyg - dyg.mean(axis=1, keepdims=True) - xhat * (dyg * xhat).mean(axis=1, keepdims=True)) / np.sqrt(var + 1e-5)
    _check("layer_norm dx", _rows_to_host(dev, dx0, lrows, LN_COLS), dx_ref, 1e-4)

    # One plain device-to-device copy of known size (logits -> dlogits, 1.648 GB each way),
    # outside every timed region: under `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE` it is the
    # calibration that the counters of the real kernels are scaled by.
    lib.mg_copy_device(dlogits.data_ptr(), logits.data_ptr(), CE_ROWS * CE_COLS * 4, st)
    dev.synchronize()

    # ---- whole step: W warm-up steps, then exactly K timed steps -------------------------
    for i in range(args.warmup):
        step(i)
    dev.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(args.warmup + i)
    dev.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- per-kernel launch durations from HIP events on the library's stream ------------
    iters = max(10, min(args.steps, 100))
    timer = EventTimer(dev, iters)
    kernels = []
    # Calibration of the HBM roofline on this box, one read-dominated and one write-only
    # stream over the same 1.65 GB buffer (outside the step): the loss-only cross-entropy reads
    # the logits once and writes 32 KB; the fill writes the buffer once.
    def ce_loss_only(i):
        lib.mg_cross_entropy_ids(logits.data_ptr(), ids.data_ptr(), loss.data_ptr(), CE_ROWS, CE_COLS, F32, I32, st)

    def fill_only(i):
        lib.mg_fill(dlogits.data_ptr(), 0.0, CE_ROWS * CE_COLS, F32, st)

    ce_read_bytes = CE_ROWS * CE_COLS * 4 + CE_ROWS * 4 + 4
    for name, fn, nbytes in (("layer_norm_fwd", ln_fwd, LN_FWD_BYTES), ("layer_norm_bwd", ln_bwd, LN_BWD_BYTES),
                             ("calibration: cross_entropy_ids, loss only (reads 1.65 GB, writes 32 KB)", ce_loss_only,
                              ce_read_bytes),
                             ("calibration: fill (writes 1.65 GB)", fill_only, CE_ROWS * CE_COLS * 4),
                             ("cross_entropy_fused_ids", ce_fused, CE_FUSED_BYTES)):
        fn(0)
        dev.synchronize()
        ts = timer.run(fn, iters)
        mean_ms = float(np.mean(ts))
        gbs = nbytes / (mean_ms * 1e-3) / 1e9
        kernels.append({"name": name, "mean_ms": round(mean_ms, 5), "median_ms": round(float(np.median(ts)), 5),
                        "algorithmic_bytes": nbytes, "achieved_GBps": round(gbs, 1),
                        "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)})
    timer.close()
    dominant = kernels[-1]

    result = {
        "metric": "fwd+bwd step ms; per-bwd-kernel HBM GB/s or MFMA % of MI355X peak",
        "value": round(ms_per_step, 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "LayerNorm fwd+bwd fp32 (2048,4096) + fused softmax-cross-entropy fwd+bwd fp32 logits "
                        "(8192,50304), int32 labels",
            "layer_norm": [LN_ROWS, LN_COLS],
            "cross_entropy": [CE_ROWS, CE_COLS],
            "labels": "int32 class ids",
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "ce_rows_kernel (mg_cross_entropy_fused_ids; the event pair also spans the one-workgroup "
                      "loss reduction that follows it)",
            "achieved": dominant["achieved_GBps"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(dominant["achieved_GBps"] / HBM_PEAK_GBS, 4),
            "traffic": _measured_traffic("ce_rows_kernel_8192x50304_f32"),
        },
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    return result


def bench_gemm16(args, dev) -> dict:
    """The 16-bit GEMM core away from the GPT step's short shapes: forward, dX and dW of a square
    bf16 Linear layer at 8192 and 4096 (no BASELINE configuration; `--workload gemm16` only, not
    part of the default run).  A step is the three products at 8192."""
    from mograd_amd import BF16, AnyBuffer

    lib, st = dev.lib, dev.stream
    P = lambda b: b.data_ptr()  # noqa: E731
    entries, keep = [], []
    for n in (8192, 4096):
        x, w, dy = (AnyBuffer.from_numpy(dev, _rng(6, 10 * i + n % 7).standard_normal(n * n, dtype=np.float32) * sc, BF16)
                    for i, sc in ((0, 1.0), (1, 0.02), (2, 1.0)))
        y, dx, dw = (AnyBuffer.create(BF16, dev, n * n) for _ in range(3))
        keep += [x, w, dy, y, dx, dw]
        fl = 2.0 * n * n * n
        entries += [
            (f"Y = X W^T bf16 {n}^3 (mg_matmul_bt)",
             lambda i, x=x, w=w, y=y, n=n: lib.mg_matmul_bt(P(x), P(w), P(y), 1, n, n, n, n, 1, n, 1, n * n, n * n, BF16, st),
             fl, "F", MFMA_BF16_PEAK_TFLOPS),
            (f"dX = dY W bf16 {n}^3 (mg_linear_bwd, dx only)",
             lambda i, x=x, w=w, dy=dy, dx=dx, n=n: lib.mg_linear_bwd(P(dy), P(x), P(w), P(dx), None, None, n, n, n, BF16, st),
             fl, "F", MFMA_BF16_PEAK_TFLOPS),
            (f"dW = dY^T X bf16 {n}^3 (mg_linear_bwd, dw only)",
             lambda i, x=x, w=w, dy=dy, dw=dw, n=n: lib.mg_linear_bwd(P(dy), P(x), P(w), None, P(dw), None, n, n, n, BF16, st),
             fl, "F", MFMA_BF16_PEAK_TFLOPS),
        ]
    # sampled rows of the 4096^3 forward against float64
    n = 4096
    x, w, y = keep[6], keep[7], keep[9]
    entries[3][1](0)
    dev.synchronize()
    rows = [0, n // 3, n - 1]
    want = x.to_numpy((n, n))[rows].astype(np.float64) @ w.to_numpy((n, n)).astype(np.float64).T
    _check("gemm16 Y = X W^T", y.to_numpy((n, n))[rows], want, 2e-2)

    def step(i):
        for e in entries[:3]:
            e[1](i)

    ms = _time_steps(dev, step, min(args.warmup, 3), min(args.steps, 20))
    kernels = _kernel_table(dev, entries, 10)
    dom = min(kernels[:3], key=lambda r: r["frac_of_mfma_peak"])
    return {
        "metric": "fwd+bwd step ms; per-bwd-kernel HBM GB/s or MFMA % of MI355X peak", "value": round(ms, 4), "unit": "ms",
        "n_gpus": 1, "steps": min(args.steps, 20), "warmup": min(args.warmup, 3), "ms_per_step": round(ms, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "bf16 Linear 8192 -> 8192 on 8192 rows: forward, dX and dW products (gemm_16bit_big_kernel), "
                               "N(0,1) activations and gradients; the same at 4096 in the kernel table"},
        "roofline": {"bound": "mfma", "kernel": "gemm_16bit_big_kernel, " + dom["name"], "achieved": dom["achieved_TFLOPs"],
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": dom["frac_of_mfma_peak"], "traffic": None},
        "kernels": kernels,
    }


# "all" runs the four BASELINE configurations; gemm16 is an extra, by name only.
WORKLOADS = {"ln_ce": bench_ln_ce, "mlp": bench_mlp, "attention": bench_attention, "gpt": bench_gpt, "gemm16": bench_gemm16}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-side baseline leg")
    ap.add_argument("--workload", choices=["all", *WORKLOADS], default="all",
                    help="all (default): every configuration in one process, the GPT training step as the headline "
                         "and the others under 'workloads'; ln_ce: LayerNorm + fused cross-entropy fp32; mlp: README "
                         "MLP fwd+bwd fp32 (matmul_bias_bt, dX, dW, db); attention: bf16 flash attention fwd+bwd; "
                         "gpt: the training step alone; gemm16: large square bf16 products (an extra, not in 'all')")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path runs on one GPU; --gpus N with N > 1 is not supported "
              "(no collective is part of the backward hot path)", file=sys.stderr)
        return 2

    from mograd_amd import Device

    dev = Device(0)
    if args.workload != "all":
        print(json.dumps(WORKLOADS[args.workload](args, dev)))
        return 0
    # Every configuration, one after the other on the same device and stream.  The headline
    # is the GPT training step; each configuration's own step time, roofline, kernel table
    # and CPU baseline sit under "workloads".
    per = {}
    for name in ("ln_ce", "mlp", "attention", "gpt"):
        print(f"[bench] {name} ...", file=sys.stderr, flush=True)
        per[name] = WORKLOADS[name](args, dev)
        dev.synchronize()
        dev.lib.mg_pool_empty_cache()
    keep = ("ms_per_step", "dtype", "config", "roofline", "kernels", "cpu_baseline", "phases_ms", "step_roofline", "whole_step",
            "via_rules", "c1_cpu")
    result = dict(per["gpt"])
    result["workloads"] = {name: {k: r[k] for k in keep if k in r} for name, r in per.items()}
    if "c1_cpu" in per["mlp"]:  # configuration 1 has no GPU leg: its CPU step time stands by itself
        result["workloads"]["c1_cpu"] = {"cpu_baseline": result["workloads"]["mlp"].pop("c1_cpu")}
    result.pop("kernels", None)  # the GPT step's table is under workloads.gpt
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
