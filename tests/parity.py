"""The closeness bar of the GPU parity tests, in one place.

The stated tolerance is elementwise: results within rtol 2e-2 in bf16 and 1e-4 in fp32 of the
reference's (the oracle's).  A bare ``|got - want| <= rtol * |want|`` cannot hold for the
elements of a tensor that are much smaller than the tensor's typical magnitude - they are sums
whose terms cancel, and carry the rounding error of terms of ordinary size - so the bound has
an absolute term tied to the tensor's scale:

    |got - want| <= rtol * (|want| + rms(want))            for every element

i.e. for bf16 (rtol 2e-2) five bf16 ulps (2^-8) of the tensor's root-mean-square value, for
fp32 1e-4 of it.  The number of elements that break the bound is reported and must be zero,
unless the caller grants a fraction (tensors whose elements are long sums of rounded
intermediates; the cap is written at the call).  The older, weaker bound on the largest error
against the largest magnitude is kept as a second assertion.

The bf16 oracle rounds where the kernels round, so agreement with it says that the device
follows the same arithmetic, not how good that arithmetic is.  `close_to_truth` is the anchor
for that: the device result may be no farther from the unrounded computation (the oracle in
float32 on the same bf16 inputs) than the bf16 oracle itself is, by a stated factor.
"""
from __future__ import annotations

import numpy as np

# Fraction of a tensor's elements that may break the elementwise bound in the stage- and
# layer-level comparisons (kernel-level comparisons grant none), and how far the worst of them
# may go.  Measured on the GPU: nothing upstream of the attention backward breaks the bound;
# downstream of it (input cotangents, QKV weight gradients) up to 7e-5 of the elements do at
# hidden 256 to 4096, by at most 2.2 x, and 4.9e-4 of the input cotangent of a layer of hidden
# 8192 with 64 heads, by at most 2.6 x, spread over rows and columns with the first tokens of
# the sequence (few keys, peaked probabilities) ahead.  The cause is the row term sum(dO * O) of the attention backward: it is
# taken from the stashed bf16 output O, and wherever the GPU's O and the oracle's differ by one
# bf16 ulp (different summation order, then rounding) every score cotangent of that row moves
# together, which no bound relative to the element's own size absorbs.
STAGE_BAD_FRAC = 1e-3
MAX_EXCESS = 4.0


def violations(got, want, rtol: float):
    """(count, total, worst excess ratio) of elements with
    |got - want| > rtol * (|want| + rms(want))."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    rms = float(np.sqrt(np.mean(want * want))) if want.size else 0.0
    bound = rtol * (np.abs(want) + rms) + 1e-300
    ratio = np.abs(got - want) / bound
    bad = ratio > 1.0
    return int(bad.sum()), int(want.size), float(ratio.max()) if want.size else 0.0


def where_bad(got, want, rtol: float) -> str:
    """For a matrix: how the violating elements spread over rows and columns (a failure that
    sits in a few whole rows or columns points at one token or one feature, not at rounding)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    if got.ndim != 2:
        return ""
    rms = float(np.sqrt(np.mean(want * want)))
    bad = np.abs(got - want) > rtol * (np.abs(want) + rms)
    rows, cols = np.nonzero(bad.any(1))[0], np.nonzero(bad.any(0))[0]
    per_row = bad.sum(1)
    top = np.argsort(-per_row)[:6]
    bins = np.histogram(np.nonzero(bad)[1], bins=16, range=(0, got.shape[1]))[0]
    return (f"; in {rows.size} of {got.shape[0]} rows and {cols.size} of {got.shape[1]} columns; "
            f"rows with most: {[(int(r), int(per_row[r])) for r in top if per_row[r]]}; "
            f"count per sixteenth of the columns: {bins.tolist()}")


def close_stage(got, want, rtol: float, what: str = ""):
    """The bar for tensors that went through whole layers (see STAGE_BAD_FRAC)."""
    close(got, want, rtol, what, STAGE_BAD_FRAC)


def close(got, want, rtol: float, what: str = "", max_bad_frac: float = 0.0,
          max_excess: float = MAX_EXCESS):
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite"
    scale = float(np.abs(want).max()) + 1e-30 if want.size else 1.0
    err = float(np.abs(got.astype(np.float64) - want.astype(np.float64)).max()) if want.size else 0.0
    assert err <= rtol * scale, f"{what}: max err {err:.4g} vs scale {scale:.4g} (rtol {rtol:g})"
    n_bad, n, worst = violations(got, want, rtol)
    # (where a fraction is granted at all, one element of a tensor too small for the fraction
    # to amount to one - a bias of 768 elements - is granted as well)
    allowed = max(max_bad_frac * n, 1.0) if max_bad_frac > 0 else 0.0
    assert n_bad <= allowed, (
        f"{what}: {n_bad} of {n} elements ({n_bad / max(n, 1):.3g}) outside "
        f"rtol {rtol:g} * (|want| + rms); worst at {worst:.3g} x the bound "
        f"(allowed fraction {max_bad_frac:g}){where_bad(got, want, rtol)}")
    assert worst <= max_excess, f"{what}: an element is {worst:.3g} x outside the elementwise bound"


# How much farther from the unrounded result than the bf16 oracle the device may be: in the
# Frobenius norm (an average over the tensor: tight), and in the largest error (one element:
# noisier, so looser).
TRUTH_FRO = 1.5
TRUTH_MAX = 2.5


def close_to_truth(got, want_bf16, want_f32, what: str = "", fro: float = TRUTH_FRO,
                   mx: float = TRUTH_MAX):
    """`got`: the device's bf16-path result; `want_bf16`: the oracle with bf16 storage rounding;
    `want_f32`: the oracle in float32 on the same (bf16-valued) inputs.  Asserts
        ||got - want_f32||_F <= fro * ||want_bf16 - want_f32||_F   and
        max|got - want_f32|  <= mx  * max|want_bf16 - want_f32|,
    each with a floor of one bf16 ulp (2^-8) of the tensor's rms / largest value per element,
    below which a bf16 result cannot be told from the truth."""
    got = np.asarray(got, np.float64)
    b = np.asarray(want_bf16, np.float64).reshape(got.shape)
    t = np.asarray(want_f32, np.float64).reshape(got.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite"
    ulp = 2.0 ** -8
    e_got, e_ref = np.linalg.norm(got - t), np.linalg.norm(b - t)
    floor_f = ulp * np.linalg.norm(t)
    assert e_got <= fro * max(e_ref, floor_f), (
        f"{what}: distance to the float32 result {e_got:.4g} (Frobenius) against the bf16 "
        f"oracle's own {e_ref:.4g}: {e_got / max(e_ref, 1e-300):.2f} x, allowed {fro} x")
    m_got, m_ref = float(np.abs(got - t).max()), float(np.abs(b - t).max())
    floor_m = ulp * float(np.abs(t).max())
    assert m_got <= mx * max(m_ref, floor_m), (
        f"{what}: largest distance to the float32 result {m_got:.4g} against the bf16 oracle's "
        f"own {m_ref:.4g}: {m_got / max(m_ref, 1e-300):.2f} x, allowed {mx} x")
