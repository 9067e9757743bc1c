"""Comparison helpers shared by the tests.

Tolerances are the reference's own: torch.isclose(rtol=1e-2, atol=2e-2) with a bounded outlier
fraction (tests/operators/utilities.py:5-41 and tests/operators/mla/test_triton.py:58,83-85 of the
reference) and 1 - cosine < 1e-5 (tests/test_ring_attention.py:92). Because attention outputs are
averages (|O| << 1 for unit-variance V), atol=2e-2 alone is weak, so every comparison also bounds
the max-abs error normalised by the oracle's max-abs value.
"""

import torch


def assert_close(actual, expected, rtol=1.6e-2, atol=1e-5, otol=0.0, what="tensor"):
    close = torch.isclose(actual.double().cpu(), expected.double().cpu(), rtol=rtol, atol=atol)
    ofrac = (~close).double().mean().item()
    if ofrac > otol:
        diff = (actual.double().cpu() - expected.double().cpu()).abs().max().item()
        raise AssertionError(
            f"{what}: not close, shape {tuple(actual.shape)}, mismatch rate {ofrac:.3%} (allowed {otol:.3%}), "
            f"greatest absolute difference {diff:.6g}"
        )


def cosine_error(a, b):
    """1 - cosine similarity: 0 = identical, 2 = opposite."""
    a, b = a.double().flatten().cpu(), b.double().flatten().cpu()
    return (1.0 - torch.dot(a, b) / (a.norm() * b.norm() + 1e-12)).item()


def norm_max_err(actual, expected):
    """max|actual - expected| / max|expected|."""
    e = expected.double().cpu()
    return ((actual.double().cpu() - e).abs().max() / e.abs().max().clamp_min(1e-30)).item()


def check_bf16_result(actual, expected, what, otol=0.0, cos_tol=1e-5, nerr_tol=2e-2):
    """bf16 kernel output against the fp64 oracle: the reference's isclose and cosine gates plus a
    normalised max-abs bound (2e-2 ~ a few bf16 ulps of the largest element, accumulated)."""
    assert torch.isfinite(actual.float()).all(), f"{what}: non-finite values"
    assert_close(actual, expected, rtol=1e-2, atol=2e-2, otol=otol, what=what)
    if expected.abs().max().item() < 1e-9:  # an exactly vanishing result (e.g. dQ of a single token)
        assert actual.float().abs().max().item() < 1e-6, f"{what}: expected zeros"
        return
    ce = cosine_error(actual, expected)
    assert ce < cos_tol, f"{what}: cosine error {ce:.3e} >= {cos_tol}"
    ne = norm_max_err(actual, expected)
    assert ne < nerr_tol, f"{what}: normalised max-abs error {ne:.3e} >= {nerr_tol}"


def check_lse(actual, expected, what, tol=1e-3):
    """fp32 base-2 LSE: max-abs error within 1e-3."""
    err = (actual.double().cpu() - expected.double().cpu()).abs().max().item()
    assert err <= tol, f"{what}: LSE max-abs error {err:.3e} > {tol}"
