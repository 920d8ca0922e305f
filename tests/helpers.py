"""Shared test helpers: seeded inputs and tolerance checks.

Inputs follow one rule everywhere: one numpy PCG64 generator per tensor, seeded with
1000 * config + tensor index, and the same host bytes go to the oracle and to the GPU.
"""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np

# Tolerances of the parity contract.
RTOL_F32, ATOL_F32 = 1e-4, 1e-5       # fp32 reductions
RTOL_BF16_ATTN = 2e-2                 # bf16 attention gradients


# bf16 attention gradients (B, S, H, D): rtol 2e-2 of the entry plus a floor for entries that
# cancel to ~0, taken per (batch, head) and not per tensor: 7.5e-3 of that head's largest entry.
# Observed on the MI355X over (B2,H3,S256,D64), (B1,H2,S1100,D64/128/256) and three heads each of
# the two benchmark shapes, causal and not: the part of |err| that rtol*|ref| does not cover is at
# most 3.8e-3 of the head's largest entry (dq, non-causal S256), typically 1-2.5e-3; the floor is
# twice the worst observation.  (|err| itself stays under 1.03e-2 of the head's largest entry.)
ATTN_BF16_FLOOR = 7.5e-3


def assert_attn_grad_close(got, ref, what, rtol=RTOL_BF16_ATTN, floor=ATTN_BF16_FLOOR, min_top=0.0):
    """|got - ref| <= rtol |ref| + floor * (largest |ref| of the same batch and head), tensors (B, S, H, D)."""
    ref = np.asarray(ref, dtype=np.float64)
    assert np.all(np.isfinite(got)), what
    top = np.maximum(np.abs(ref).max(axis=(1, 3), keepdims=True), min_top)
    bound = rtol * np.abs(ref) + floor * top
    worst = float(np.max(np.abs(got - ref) / bound))
    assert worst <= 1.0, f"{what}: worst |err| / (rtol |ref| + floor * head max) = {worst:.3g}"


def rng_for(config: int, tensor: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(1000 * config + tensor))


def normal(config, tensor, shape, std=1.0, mean=0.0):
    return (rng_for(config, tensor).standard_normal(shape) * std + mean).astype(np.float32)


def uniform(config, tensor, shape, lo, hi):
    return rng_for(config, tensor).uniform(lo, hi, shape).astype(np.float32)


def integers(config, tensor, shape, lo, hi, dtype=np.int32):
    return rng_for(config, tensor).integers(lo, hi, shape).astype(dtype)


def worst_violation(got, want, rtol, atol):
    """max over elements of |got - want| / (atol + rtol * |want|); <= 1 passes."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    if not np.all(np.isfinite(got)):
        return float("inf")
    if not got.size:
        return 0.0
    err = np.abs(got - want)
    bound = atol + rtol * np.abs(want)
    ratio = np.divide(err, bound, out=np.where(err > 0, np.inf, 0.0), where=bound > 0)
    return float(np.max(ratio))


def assert_close(got, want, rtol, atol, what=""):
    v = worst_violation(got, want, rtol, atol)
    assert v <= 1.0, f"{what}: worst |err| / (atol + rtol*|want|) = {v:.3g} (rtol={rtol}, atol={atol})"


def assert_sum_close(got, want, term_l1, rtol=RTOL_F32, atol=ATOL_F32, what=""):
    """For an fp32 sum of many terms (column sums, dot products of a matmul).

    The parity tolerance rtol/atol applies to the value; on top of it the absolute floor
    is never below 16 * 2^-24 * sum|terms|: an fp32 accumulator cannot resolve less than
    about one unit roundoff of the mass it has summed, so a result that cancelled to near
    zero is held to the rounding of its summands, not of itself.  `term_l1` is that mass
    per output element.
    """
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    floor = np.maximum(atol, 16.0 * 2.0 ** -24 * np.asarray(term_l1, dtype=np.float64))
    err = np.abs(got - want)
    bound = floor + rtol * np.abs(want)
    worst = float(np.max(err / bound))
    assert np.all(np.isfinite(got)) and worst <= 1.0, f"{what}: worst err/bound = {worst:.3g}"


def golden(section: str) -> list:
    """Entries of one section of tests/golden/reference_vectors.json: the golden vectors the
    reference's own tests hold for this path (inputs, expected outputs, tolerance, citation)."""
    with open(Path(__file__).resolve().parent / "golden" / "reference_vectors.json") as f:
        return json.load(f)[section]
