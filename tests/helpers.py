"""Shared helpers of the parity tests: seeded inputs and the tolerance rules.

Tolerances (stated once, used everywhere):
  * float32 results: rtol 1e-5 / atol 1e-6 against the float64 closed form;
  * sums/means additionally get the a-priori summation bound (n-1)*2^-24*sum|x| — a float32
    sum near zero cannot be relatively accurate in ANY order, and the reference's own tests
    (assert_close vs torch CPU) never probe that regime;
  * bfloat16 / float16 results: the float32 rule applied before the final cast, i.e. the result
    must equal the correctly rounded closed form up to one unit in the last place of the
    storage type (rtol 2^-8 for bf16, 2^-11 for fp16) plus the float32 slack;
  * bf16 GEMM: relative Frobenius error <= 1e-2 against float64 of the same rounded inputs;
  * argmax / integer results: exact.
"""

import numpy as np
import torch

FP32_RTOL, FP32_ATOL = 1e-5, 1e-6
ULP = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}


def seeded(shape, seed=0, scale=1.0, dtype=torch.float32, shift=0.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32) * scale + shift
    return x.to(dtype)


def as64(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().to(torch.float64).numpy()


def assert_close64(got: torch.Tensor, want64: np.ndarray, *, rtol=FP32_RTOL, atol=FP32_ATOL,
                   extra_abs=None, what="", rounded_want=False):
    """|got - want| <= atol + rtol*|want| + half a storage ulp of |want| (+ extra_abs).

    ``ULP`` holds the largest relative half-spacing of the storage type. Set ``rounded_want``
    when ``want64`` was itself rounded to the storage type (another implementation's output):
    two correctly rounded results of nearly equal exact values may differ by one full spacing,
    which is up to four times that figure."""
    g = as64(got)
    assert g.shape == want64.shape, f"{what}: shape {g.shape} vs {want64.shape}"
    ulp = ULP[got.dtype] * (4.0 if rounded_want else 1.0)
    tol = atol + (rtol + ulp) * np.abs(want64)
    if extra_abs is not None:
        tol = tol + extra_abs
    both_nan = np.isnan(g) & np.isnan(want64)
    same_inf = np.isinf(g) & np.isinf(want64) & (np.sign(g) == np.sign(want64))
    err = np.abs(g - want64)
    bad = ~(both_nan | same_inf) & ~(err <= tol)
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err - tol, -np.inf)), g.shape)
        raise AssertionError(
            f"{what}: {bad.sum()} of {g.size} elements out of tolerance; worst at {i}: "
            f"got {g[i]!r} want {want64[i]!r} err {err[i]:.3e} tol {tol[i]:.3e}")


def rel_frobenius(got: torch.Tensor, want64: np.ndarray) -> float:
    g = as64(got)
    return float(np.linalg.norm(g - want64) / max(np.linalg.norm(want64), 1e-300))
