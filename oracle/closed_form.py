"""Float64 closed forms of the hot ops — TEST INFRASTRUCTURE (see ``oracle/__init__.py``).

These are the textbook definitions evaluated in float64 with numpy; the parity tests measure
both the C oracle and the HIP kernels against them. Inputs are numpy arrays (any float dtype;
bf16 tensors are widened by the caller), outputs are float64 (int64 for argmax).
"""

from __future__ import annotations

import numpy as np


def softmax(x: np.ndarray, axis: int = -1) -> np.ndarray:
    x = x.astype(np.float64)
    e = np.exp(x - x.max(axis=axis, keepdims=True))
    return e / e.sum(axis=axis, keepdims=True)


def softmax_scaled_causal(x: np.ndarray, scale: float, causal: bool) -> np.ndarray:
    """float64 softmax(x*scale) over the last axis of [..., q, cols]; causal keeps j <= query row."""
    z = x.astype(np.float64) * scale
    if causal:
        q, cols = z.shape[-2], z.shape[-1]
        keep = np.arange(cols)[None, :] <= np.arange(q)[:, None]
        z = np.where(keep, z, -np.inf)
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, causal: bool) -> np.ndarray:
    """float64 softmax(scale q k^T [+ causal]) v for [B,H,T,D],[B,H,S,D],[B,H,S,D] -> [B,T,H,D]."""
    s = np.einsum("bhtd,bhsd->bhts", q.astype(np.float64), k.astype(np.float64))
    p = softmax_scaled_causal(s, scale, causal)
    return np.einsum("bhts,bhsd->bthd", p, v.astype(np.float64))


def log_softmax(x: np.ndarray, axis: int = -1) -> np.ndarray:
    x = x.astype(np.float64)
    s = x - x.max(axis=axis, keepdims=True)
    return s - np.log(np.exp(s).sum(axis=axis, keepdims=True))


def layer_norm(x: np.ndarray, gamma, beta, eps: float):
    """Biased variance over the last axis; returns (out, mean, rstd) with keepdim statistics."""
    x = x.astype(np.float64)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    rstd = 1.0 / np.sqrt(var + eps)
    out = (x - mean) * rstd
    if gamma is not None:
        out = out * gamma.astype(np.float64)
    if beta is not None:
        out = out + beta.astype(np.float64)
    return out, mean, rstd


def gelu_tanh(x: np.ndarray) -> np.ndarray:
    x = x.astype(np.float64)
    return 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))


def gelu_erf(x: np.ndarray) -> np.ndarray:
    from scipy.special import erf

    x = x.astype(np.float64)
    return 0.5 * x * (1.0 + erf(x / np.sqrt(2.0)))


def gemm(a: np.ndarray, b: np.ndarray, bias=None) -> np.ndarray:
    out = a.astype(np.float64) @ b.astype(np.float64)
    if bias is not None:
        out = out + bias.astype(np.float64)
    return out


def argmax_first(x: np.ndarray, axis: int = -1) -> np.ndarray:
    """First occurrence of the maximum; NaN counts as the maximum (numpy and ATen agree)."""
    return np.argmax(x, axis=axis).astype(np.int64)


def sum_error_bound(x: np.ndarray, axis=-1, eps: float = 2.0 ** -24) -> np.ndarray:
    """A priori bound on |fl(sum) - sum| for ANY summation order of n fp32 terms:
    (n-1) * eps * sum|x_i| (Higham, Accuracy and Stability of Numerical Algorithms, eq. 4.4)."""
    x = np.abs(x.astype(np.float64))
    n = x.shape[axis] if axis is not None else x.size
    return (n - 1) * eps * x.sum(axis=axis)
