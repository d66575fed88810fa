"""Shared helpers for the test-suite: seeded inputs the way the reference's own test builds
them (tests/test_streaming_attention.py:78-150) and the comparison bars."""
from __future__ import annotations

import numpy as np
import torch

# parity bars: fp32 <= 1e-4 abs; bf16/fp16 <= 2e-2 abs + 1e-2 rel against the fp32/f64 oracle
TOL = {torch.float32: (1e-4, 0.0), torch.float16: (2e-2, 1e-2), torch.bfloat16: (2e-2, 1e-2)}


# The log-sum-exp is a float32 output whatever the input type: scores are accumulated in float32 from the
# (exactly representable) 16-bit inputs, scaled in float32, and the probabilities are summed in float32
# before they are rounded for the second product, so the bar is the float32 one for every type.
LSE_ATOL = {torch.float32: 1e-4, torch.float16: 1e-4, torch.bfloat16: 1e-4}


def make_inputs(B, H, T, D, seed=20, dtype=torch.float32):
    """q, k, v, dO ~ N(0,1) from a seeded CPU generator, rounded to ``dtype`` (the values the
    kernel will actually see), returned as CPU tensors of that dtype."""
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(B, H, T, D, generator=g).to(dtype) for _ in range(4)]


def tricky_lens(B, T, C, R, seed=20):
    """Lengths around the chunk size, the window size, T and T+1 (> T must clamp), as in
    tests/test_streaming_attention.py:117-135 but drawn from a seeded generator."""
    cand = [2, 5, C, C + 1, max(C - 1, 1), max(C // 2, 1), C // 2 + C, max(C * R, 1), C * R + 1,
            max(C * R - 1, 1), T + 1, T, max(T // 2, 1), max(T // 4, 1)]
    cand = [min(max(int(x), 1), 2**31 - 1) for x in cand]
    rng = np.random.default_rng(seed)
    return torch.tensor(rng.choice(cand, B), dtype=torch.int32)


def assert_close(name, got, want, dtype):
    atol, rtol = TOL[dtype]
    got = torch.as_tensor(got).detach().double().cpu()
    want = torch.as_tensor(want).detach().double().cpu()
    assert got.shape == want.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    bad = err > bound
    assert not bad.any(), (
        f"{name}: {int(bad.sum())} elements out of tolerance, max abs err {err.max().item():.3e} "
        f"(atol {atol}, rtol {rtol}), worst at {np.unravel_index(int(err.argmax()), err.shape)}"
    )


def assert_close_lse(got, want, dtype):
    """Absolute bar of the float32 log-sum-exp output (LSE_ATOL), whatever the input type."""
    got = torch.as_tensor(got).detach().double().cpu()
    want = torch.as_tensor(want).detach().double().cpu()
    assert got.shape == want.shape and torch.isfinite(got).all()
    err = (got - want).abs().max().item() if got.numel() else 0.0
    assert err <= LSE_ATOL[dtype], f"LSE: max abs err {err:.3e} > {LSE_ATOL[dtype]} for {dtype} inputs"


def error_report(got, want):
    """(max abs error, max error relative to max |want|, relative Frobenius error)."""
    got = torch.as_tensor(got).detach().double().cpu()
    want = torch.as_tensor(want).detach().double().cpu()
    err = (got - want).abs()
    scale = want.abs().max().item() or 1.0
    fro = want.norm().item() or 1.0
    return err.max().item(), err.max().item() / scale, (got - want).norm().item() / fro


def assert_close_rounding_aware(name, got, exact, rounded, dtype):
    """The BASELINE bar widened by the error that rounding P and dS to ``dtype`` causes in a
    float64 evaluation of the same formulas: bound = atol + rtol * |exact| + 2 * max |rounded - exact|,
    the maximum taken over the element's own (batch, head) slice.  The allowance cannot be narrower than
    that: the largest part of a row's deviation is one random number per row (the error of delta, which
    multiplies the whole row of dS), so a single row of the float64 evaluation says little about the same
    row of another evaluation with other rounding errors, while the rows of one head are samples of the
    same distribution.  A wrong element in another head or batch entry gets no cover from it."""
    atol, rtol = TOL[dtype]
    got = torch.as_tensor(got).detach().double().cpu()
    exact = torch.as_tensor(exact).detach().double().cpu()
    rounded = torch.as_tensor(rounded).detach().double().cpu()
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    allowance = 2.0 * (rounded - exact).abs().amax((-2, -1), keepdim=True)
    err = (got - exact).abs()
    bad = err > atol + rtol * exact.abs() + allowance
    assert not bad.any(), (
        f"{name}: {int(bad.sum())} elements out of tolerance, max abs err {err.max().item():.3e} "
        f"(atol {atol}, rtol {rtol}, largest per-head rounding allowance {allowance.max().item():.3e})")
