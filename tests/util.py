"""Shared helpers for the parity tests: seeded inputs, tolerances, comparisons."""
from __future__ import annotations

import numpy as np
import torch

# Tolerances of the parity bar: max |a-b| / max(1, |b|).
TOL = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 2e-2}
# Bounds of the one-normalisation comparison (assert_scaled_close): half the element-wise bar for 16-bit storage
# (the worst error any attention or cut-cross-entropy case shows is 5.5e-3 of the tensor's scale).
STOL = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 1e-2}
DTYPES = [torch.float32, torch.float16, torch.bfloat16]
DTYPE_IDS = ["f32", "f16", "bf16"]


def randn(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def randint(high, shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, high, shape, generator=g, dtype=torch.int32)


def to_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().to(torch.float64).numpy()


def rel_err(actual, expected) -> float:
    a = to_np(actual) if isinstance(actual, torch.Tensor) else np.asarray(actual, dtype=np.float64)
    e = to_np(expected) if isinstance(expected, torch.Tensor) else np.asarray(expected, dtype=np.float64)
    assert a.shape == e.shape, (a.shape, e.shape)
    if a.size == 0:
        return 0.0
    assert np.isfinite(a).all(), "non-finite values in result"
    return float(np.max(np.abs(a - e) / np.maximum(1.0, np.abs(e))))


def assert_close(actual, expected, tol, what=""):
    err = rel_err(actual, expected)
    assert err <= tol, f"{what}: max rel err {err:.3e} > {tol:.1e}"


def assert_scaled_close(actual, expected, tol, what=""):
    """One normalisation only: max |a-b| <= tol * max(1, max |expected|). For results that are sums of many
    rounded terms (dK/dV, dW, dC), whose rounding error follows the tensor's scale and not each element's.
    Prints the observed error so that a run shows how far inside the bound the kernels are."""
    a = to_np(actual) if isinstance(actual, torch.Tensor) else np.asarray(actual, dtype=np.float64)
    e = to_np(expected) if isinstance(expected, torch.Tensor) else np.asarray(expected, dtype=np.float64)
    assert a.shape == e.shape, (a.shape, e.shape)
    if a.size == 0:
        return
    assert np.isfinite(a).all(), f"{what}: non-finite values in result"
    scale = max(1.0, float(np.abs(e).max()))
    err = float(np.abs(a - e).max()) / scale
    print(f"[parity] {what}: max|a-b|/max(1,max|w|) = {err:.3e} (bound {tol:.1e}, scale {scale:.3g})")
    assert err <= tol, f"{what}: max abs err / scale {err:.3e} > {tol:.1e} (scale {scale:.3e})"


def scaled_tol(dtype, expected, floor=1.0):
    """Tolerance for results that are sums of many rounded terms: TOL times the result's scale."""
    e = to_np(expected) if isinstance(expected, torch.Tensor) else np.asarray(expected, dtype=np.float64)
    return TOL[dtype] * max(floor, float(np.abs(e).max()) if e.size else 1.0)


def bits(t: torch.Tensor) -> np.ndarray:
    """Raw storage bits, for bit-exact comparisons."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy()
    return t.view(torch.int16).numpy()
