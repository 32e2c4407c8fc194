"""CPU oracle for the hot ATen ops — TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import
this package. Nothing under ``torch-max-backend_amd/`` imports it, and the product raises when
its HIP library is missing instead of falling back to anything here.

Three layers, each checked against the others by ``tests/test_oracle_pins.py``:

* ``tmb_oracle.c`` (loaded below through ctypes): the reference's CPU kernel bodies restated in
  C — fp32 sequential arithmetic, one cast (citations in that file's header);
* ``oracle.closed_form``: float64 numpy closed forms (the mathematical truth the tolerances of
  the parity tests are measured against);
* the ``aten_*`` functions in this module: the ATen-level semantics of the reference's mapping
  functions (dim normalisation, keepdim, dtype promotion, output shapes), following
  ``torch_mojo_backend/aten_functions.py`` at the lines each docstring cites, evaluated with the
  C kernels above on CPU tensors.

Parity with the bit patterns of Modular MAX's own CPU kernels (``max`` 26.5.0.dev2026072306, a
third-party dependency that is not in the reference tree) is **parity unpinned**; what is pinned
is agreement with PyTorch CPU eager at ``assert_close`` tolerances, which is the only comparison
the reference's tests make (``torch_mojo_backend/testing.py:186-229``).
"""

from __future__ import annotations

import ctypes
import math
import os
import subprocess
from typing import Optional, Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtmb_oracle.so")

F32, F16, BF16, I64, I32 = 0, 1, 2, 3, 4
SUM, MEAN, AMAX = 0, 1, 2
EPI_NONE, EPI_GELU_TANH, EPI_GELU_ERF = 0, 1, 2

_DTYPE_CODES = {
    torch.float32: F32,
    torch.float16: F16,
    torch.bfloat16: BF16,
    torch.int64: I64,
    torch.int32: I32,
}
_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def build(force: bool = False) -> str:
    """Compile ``tmb_oracle.c`` into ``libtmb_oracle.so`` (gcc, about a second)."""
    src = os.path.join(_HERE, "tmb_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B", "libtmb_oracle.so"], check=True,
                       capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, vp, ci, dbl = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_double
        L.orc_gemm.argtypes = [vp, vp, vp, vp] + [i64] * 10 + [ci] * 4
        L.orc_gemm_residual.argtypes = [vp, vp, vp, vp, vp] + [i64] * 12 + [ci] * 6
        L.orc_gemm_residual.restype = ci
        L.orc_layer_norm_mixed.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, dbl, ci, ci]
        L.orc_layer_norm_mixed.restype = ci
        L.orc_softmax.argtypes = [vp, vp, i64, i64, ci, ci, ci]
        L.orc_softmax_scaled.argtypes = [vp, vp, i64, i64, ci, ctypes.c_float, ci, i64]
        L.orc_softmax_scaled.restype = ci
        L.orc_attention.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, ctypes.c_float, ci, ci]
        L.orc_attention.restype = ci
        L.orc_attention_lse.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, ctypes.c_float, ci, ci]
        L.orc_attention_lse.restype = ci
        L.orc_attention_backward.argtypes = [vp] * 9 + [i64] * 5 + [ctypes.c_float, ci, ci]
        L.orc_attention_backward.restype = ci
        L.orc_layer_norm.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, dbl, ci]
        L.orc_reduce.argtypes = [vp, vp, i64, i64, ci, ci]
        L.orc_argmax.argtypes = [vp, vp, i64, i64, ci]
        L.orc_gelu.argtypes = [vp, vp, i64, ci, ci]
        L.orc_gelu_backward.argtypes = [vp, vp, vp, i64, ci, ci]
        L.orc_gather_rows.argtypes = [vp, vp, vp, i64, i64, i64, ci, ci]
        L.orc_gather_rows.restype = ci
        L.orc_softmax_backward.argtypes = [vp, vp, vp, i64, i64, ci, ci]
        L.orc_layer_norm_backward.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, ci, vp]
        L.orc_nll_log_softmax_backward.argtypes = [vp, vp, vp, vp, vp, i64, i64, ci, i64, ci, vp]
        for f in (L.orc_gelu_backward, L.orc_softmax_backward, L.orc_layer_norm_backward):
            f.restype = ci
        L.orc_convert_to_f32.argtypes = [vp, vp, i64, ci]
        L.orc_convert_from_f32.argtypes = [vp, vp, i64, ci]
        for f in (L.orc_gemm, L.orc_softmax, L.orc_layer_norm, L.orc_reduce, L.orc_argmax,
                  L.orc_gelu):
            f.restype = ci
        L.orc_convert_to_f32.restype = None
        L.orc_convert_from_f32.restype = None
        _lib = L
    return _lib


def _code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise TypeError(f"oracle: unsupported dtype {dtype}") from None


def _cpu(t: torch.Tensor) -> torch.Tensor:
    assert t.device.type == "cpu", "the oracle only takes CPU tensors"
    return t.contiguous()


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"oracle {what} failed with code {rc}")


# ---------------------------------------------------------------------------
# Row-level kernels (thin wrappers over the C functions)
# ---------------------------------------------------------------------------
EPI_ROUND_LIKE_UNFUSED = 0x100


def gemm(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None, *,
         epilogue: int = EPI_NONE, residual: Optional[torch.Tensor] = None,
         out_dtype: Optional[torch.dtype] = None, round_like_unfused: bool = False) -> torch.Tensor:
    """``epilogue(a @ b + bias) [+ residual]`` for 2-D or 3-D (batched) operands of any strides,
    formed in float32 and cast once (matmul_ops.mojo:2651-2657); ``round_like_unfused`` rounds
    to the operands' dtype after the bias and after the GELU, as separate kernels would.
    ``residual`` has the result's shape and the operands' dtype or float32; ``out_dtype``
    defaults to the operands' dtype.

    Strided views are passed through as they are (transpose flags / leading dimensions) when
    each matrix is dense row-major or dense column-major, otherwise materialised first.
    """
    assert a.dtype == b.dtype and a.dtype in _FLOATS
    batched = a.dim() == 3
    if not batched:
        a3, b3 = a.unsqueeze(0), b.unsqueeze(0)
    else:
        a3, b3 = a, b
    assert a3.dim() == 3 and b3.dim() == 3 and a3.shape[0] == b3.shape[0]
    assert a3.shape[2] == b3.shape[1]
    batch, m, k = a3.shape
    n = b3.shape[2]

    def layout(t):
        rows, cols = t.shape[1], t.shape[2]
        sb, sr, sc = t.stride()
        if sc == 1 and sr >= max(cols, 1):
            return t, 0, sr, sb
        if sr == 1 and sc >= max(rows, 1):
            return t, 1, sc, sb
        t = t.contiguous()
        return t, 0, max(cols, 1), t.stride(0)

    a3, ta, lda, sa = layout(a3)
    b3, tb, ldb, sb = layout(b3)
    out = torch.empty((batch, m, n), dtype=out_dtype or a.dtype)
    if bias is not None:
        assert bias.dtype == a.dtype and tuple(bias.shape) == (n,)
        bias = _cpu(bias)
    res = None
    if residual is not None:
        res = _cpu(residual).reshape(batch, m, n).contiguous()
        assert res.dtype in (a.dtype, torch.float32)
    flags = epilogue | (EPI_ROUND_LIKE_UNFUSED if round_like_unfused else 0)
    if out.numel():
        _check(lib().orc_gemm_residual(
            out.data_ptr(), a3.data_ptr(), b3.data_ptr(), _ptr(bias), _ptr(res), batch, m, n, k,
            lda, ldb, n, n, sa, sb, m * n, m * n, ta, tb, _code(a.dtype),
            _code(res.dtype if res is not None else a.dtype), _code(out.dtype), flags), "gemm")
    return out if batched else out[0]


def softmax_rows(x: torch.Tensor, *, log: bool = False,
                 out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    x = _cpu(x)
    assert x.dim() == 2
    out = torch.empty(x.shape, dtype=out_dtype or x.dtype)
    if x.numel():
        _check(lib().orc_softmax(out.data_ptr(), x.data_ptr(), x.shape[0], x.shape[1],
                                 _code(x.dtype), _code(out.dtype), int(log)), "softmax")
    return out


def softmax_scaled(x: torch.Tensor, scale: float, causal_q_len: int = 0,
                   round_scaled: bool = False) -> torch.Tensor:
    """softmax(x*scale) over the last dim; rows are flattened, causal rows keep j <= r % q_len."""
    x = _cpu(x).contiguous()
    out = torch.empty_like(x)
    cols = x.shape[-1]
    if x.numel():
        _check(lib().orc_softmax_scaled(out.data_ptr(), x.data_ptr(), x.numel() // cols, cols,
                                        _code(x.dtype), float(scale), int(bool(round_scaled)),
                                        int(causal_q_len)), "softmax_scaled")
    return out


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
              causal: bool) -> torch.Tensor:
    """[B,H,T,D] x [B,H,S,D] x [B,H,S,D] -> [B,T,H,D], stage by stage like the unfused graph."""
    q, k, v = (_cpu(x).contiguous() for x in (q, k, v))
    b, h, t, d = q.shape
    out = torch.empty((b, t, h, d), dtype=q.dtype)
    if out.numel():
        _check(lib().orc_attention(out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), b, h,
                                   t, k.shape[2], d, float(scale), int(bool(causal)),
                                   _code(q.dtype)), "attention")
    return out


def attention_lse(q: torch.Tensor, k: torch.Tensor, scale: float, causal: bool) -> torch.Tensor:
    """[B,H,T,D] x [B,H,S,D] -> float32 [B,H,T]: log-sum-exp of each query's scaled scores."""
    q, k = _cpu(q).contiguous(), _cpu(k).contiguous()
    b, h, t, d = q.shape
    lse = torch.empty((b, h, t), dtype=torch.float32)
    if lse.numel():
        _check(lib().orc_attention_lse(lse.data_ptr(), q.data_ptr(), k.data_ptr(), b, h, t,
                                       k.shape[2], d, float(scale), int(bool(causal)),
                                       _code(q.dtype)), "attention_lse")
    return lse


def attention_backward(dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                       out: torch.Tensor, lse: torch.Tensor, scale: float, causal: bool):
    """Gradients (dq, dk, dv), each [B,H,T|S,D], of `attention`'s [B,T,H,D] output given its
    gradient `dout` (same layout) and the float32 [B,H,T] log-sum-exp."""
    q, k, v, out, dout = (_cpu(x).contiguous() for x in (q, k, v, out, dout))
    lse = _cpu(lse).contiguous().float()
    b, h, t, d = q.shape
    assert tuple(out.shape) == (b, t, h, d) and tuple(dout.shape) == (b, t, h, d)
    dq, dk, dv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
    if q.numel() and k.numel():
        _check(lib().orc_attention_backward(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                            dout.data_ptr(), q.data_ptr(), k.data_ptr(),
                                            v.data_ptr(), out.data_ptr(), lse.data_ptr(), b, h, t,
                                            k.shape[2], d, float(scale), int(bool(causal)),
                                            _code(q.dtype)), "attention_backward")
    return dq, dk, dv


def layer_norm_rows(x: torch.Tensor, gamma: Optional[torch.Tensor], beta: Optional[torch.Tensor],
                    eps: float, out_dtype: Optional[torch.dtype] = None):
    x = _cpu(x)
    assert x.dim() == 2
    rows, cols = x.shape
    out = torch.empty(x.shape, dtype=out_dtype or x.dtype)
    mean = torch.empty(rows, dtype=torch.float32)
    rstd = torch.empty(rows, dtype=torch.float32)
    g = None if gamma is None else _cpu(gamma.reshape(-1))
    b = None if beta is None else _cpu(beta.reshape(-1))
    assert all(p is None or p.dtype == out.dtype for p in (g, b))
    if x.numel():
        _check(lib().orc_layer_norm_mixed(out.data_ptr(), mean.data_ptr(), rstd.data_ptr(),
                                          x.data_ptr(), _ptr(g), _ptr(b), rows, cols, float(eps),
                                          _code(x.dtype), _code(out.dtype)), "layer_norm")
    return out, mean, rstd


def reduce_rows(x: torch.Tensor, op: int) -> torch.Tensor:
    x = _cpu(x)
    assert x.dim() == 2
    out = torch.empty(x.shape[0], dtype=x.dtype)
    if x.shape[0]:
        _check(lib().orc_reduce(out.data_ptr(), x.data_ptr(), x.shape[0], x.shape[1], op,
                                _code(x.dtype)), "reduce")
    return out


def argmax_rows(x: torch.Tensor) -> torch.Tensor:
    x = _cpu(x)
    assert x.dim() == 2
    out = torch.empty(x.shape[0], dtype=torch.int64)
    if x.shape[0]:
        _check(lib().orc_argmax(out.data_ptr(), x.data_ptr(), x.shape[0], x.shape[1],
                                _code(x.dtype)), "argmax")
    return out


def gelu(x: torch.Tensor, approximate: str = "none") -> torch.Tensor:
    x = _cpu(x)
    out = torch.empty_like(x)
    if x.numel():
        _check(lib().orc_gelu(out.data_ptr(), x.data_ptr(), x.numel(), _code(x.dtype),
                              int(approximate == "tanh")), "gelu")
    return out


def embedding(table: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """``table[indices]`` (reference: nn_ops.mojo:1153-1176 through aten_fast.py:5336-5371)."""
    table, indices = _cpu(table).contiguous(), _cpu(indices).contiguous()
    out = torch.empty(tuple(indices.shape) + (table.shape[1],), dtype=table.dtype)
    if out.numel():
        _check(lib().orc_gather_rows(out.data_ptr(), table.data_ptr(), indices.data_ptr(),
                                     indices.numel(), table.shape[1], table.shape[0],
                                     _code(table.dtype), 3 if indices.dtype == torch.int64 else 4),
               "embedding")
    return out


def gelu_backward(grad: torch.Tensor, x: torch.Tensor, approximate: str = "none") -> torch.Tensor:
    grad, x = _cpu(grad), _cpu(x)
    out = torch.empty_like(x)
    if x.numel():
        _check(lib().orc_gelu_backward(out.data_ptr(), grad.data_ptr(), x.data_ptr(), x.numel(),
                                       _code(x.dtype), int(approximate == "tanh")), "gelu_backward")
    return out


def softmax_backward_rows(grad: torch.Tensor, out: torch.Tensor, log: bool) -> torch.Tensor:
    grad, out = _cpu(grad), _cpu(out)
    assert out.dim() == 2 and grad.shape == out.shape
    res = torch.empty_like(out)
    if out.numel():
        _check(lib().orc_softmax_backward(res.data_ptr(), grad.data_ptr(), out.data_ptr(),
                                          out.shape[0], out.shape[1], _code(out.dtype), int(log)),
               "softmax_backward")
    return res


def nll_log_softmax_backward(grad_out: torch.Tensor, logp: torch.Tensor, target: torch.Tensor,
                             total_weight: torch.Tensor, reduction: int, ignore_index: int) -> torch.Tensor:
    """What ``nll_loss_backward`` followed by ``_log_softmax_backward_data`` hands to the logits
    (reference: eager_kernels/loss_ops.mojo:234-311, aten_functions.py:788-833)."""
    grad_out, logp, target = _cpu(grad_out).to(logp.dtype), _cpu(logp), _cpu(target)
    total_weight = _cpu(total_weight).to(logp.dtype)
    assert logp.dim() == 2 and target.dtype == torch.int64 and target.shape == (logp.shape[0],)
    res = torch.empty_like(logp)
    scratch = torch.empty_like(logp)
    if logp.numel():
        _check(lib().orc_nll_log_softmax_backward(
            res.data_ptr(), logp.data_ptr(), target.data_ptr(), grad_out.contiguous().data_ptr(),
            total_weight.contiguous().data_ptr(), logp.shape[0], logp.shape[1], int(reduction),
            int(ignore_index), _code(logp.dtype), scratch.data_ptr()), "nll_log_softmax_backward")
    return res


def layer_norm_backward_rows(grad: torch.Tensor, x: torch.Tensor, mean: torch.Tensor,
                             rstd: torch.Tensor, gamma: Optional[torch.Tensor]):
    """(dx, dgamma, dbeta) for [rows, cols] inputs and float32 per-row statistics."""
    grad, x = _cpu(grad), _cpu(x)
    assert x.dim() == 2 and grad.shape == x.shape
    rows, cols = x.shape
    mean = _cpu(mean.reshape(-1).float())
    rstd = _cpu(rstd.reshape(-1).float())
    g = None if gamma is None else _cpu(gamma.reshape(-1))
    dx = torch.empty_like(x)
    dg = torch.empty(cols, dtype=x.dtype)
    db = torch.empty(cols, dtype=x.dtype)
    scratch = torch.empty(2 * cols, dtype=torch.float32)
    _check(lib().orc_layer_norm_backward(dx.data_ptr(), dg.data_ptr(), db.data_ptr(), grad.data_ptr(),
                                         x.data_ptr(), mean.data_ptr(), rstd.data_ptr(), _ptr(g),
                                         rows, cols, _code(x.dtype), scratch.data_ptr()),
           "layer_norm_backward")
    return dx, dg, db


# ---------------------------------------------------------------------------
# ATen-level semantics (reference: torch_mojo_backend/aten_functions.py)
# ---------------------------------------------------------------------------
def _move_last(x: torch.Tensor, dim: int) -> torch.Tensor:
    return x.movedim(dim, -1).contiguous()


def aten__softmax(x: torch.Tensor, dim: int, half_to_float: bool) -> torch.Tensor:
    """aten_functions.py:681-714: ``half_to_float`` computes and returns float32."""
    out_dtype = torch.float32 if half_to_float else x.dtype
    if x.dim() == 0:
        return torch.ones((), dtype=out_dtype)
    dim %= x.dim()
    moved = _move_last(x, dim)
    rows = moved.reshape(-1, moved.shape[-1])
    out = softmax_rows(rows, out_dtype=out_dtype).reshape(moved.shape)
    return out.movedim(-1, dim)


def aten__log_softmax(x: torch.Tensor, dim: int, half_to_float: bool) -> torch.Tensor:
    """aten_functions.py:718-785: ``half_to_float`` is only legal for float16 input."""
    if half_to_float and x.dtype != torch.float16:
        raise ValueError(
            f"half_to_float conversion is supported for Half (float16) type only, got {x.dtype}")
    out_dtype = torch.float32 if half_to_float else x.dtype
    if x.dim() == 0:
        return torch.zeros((), dtype=out_dtype)
    dim %= x.dim()
    moved = _move_last(x, dim)
    rows = moved.reshape(-1, moved.shape[-1])
    out = softmax_rows(rows, log=True, out_dtype=out_dtype).reshape(moved.shape)
    return out.movedim(-1, dim)


def aten_native_layer_norm(x: torch.Tensor, normalized_shape: Sequence[int],
                           weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                           eps: float):
    """aten_functions.py:2829-2868 / aten_fast.py:2704-2794: (out, mean, rstd) with float32
    keepdim statistics of shape ``x.shape[:-k] + (1,)*k``."""
    k = len(normalized_shape)
    assert tuple(x.shape[-k:]) == tuple(normalized_shape)
    cols = math.prod(normalized_shape)
    rows = x.numel() // max(cols, 1)
    out, mean, rstd = layer_norm_rows(x.contiguous().reshape(rows, cols), weight, bias, eps)
    stat_shape = tuple(x.shape[:-k]) + (1,) * k
    return out.reshape(x.shape), mean.reshape(stat_shape), rstd.reshape(stat_shape)


def _norm_dims(dim, rank: int) -> list:
    """aten_fast.py:2944-2973: None or [] mean "all"; negatives wrap; result sorted unique."""
    if dim is None:
        return list(range(rank))
    if isinstance(dim, int):
        dim = [dim]
    dims = list(dim)
    if not dims:
        return list(range(rank))
    out = sorted({d % rank for d in dims}) if rank else []
    assert len(out) == len(dims), "duplicate reduce dims"
    return out


def _reduce(x: torch.Tensor, dims: list, keepdim: bool, op: int) -> torch.Tensor:
    """Geometry of op_utils/__init__.mojo:651-720: kept dims (ascending) then reduce dims."""
    rank = x.dim()
    kept = [d for d in range(rank) if d not in dims]
    perm = kept + dims
    moved = x.permute(perm).contiguous() if rank else x.reshape(1)
    cols = math.prod(x.shape[d] for d in dims) if rank else 1
    rows = moved.numel() // max(cols, 1)
    out = reduce_rows(moved.reshape(rows, cols), op)
    kept_shape = [x.shape[d] for d in kept]
    out = out.reshape(kept_shape)
    if keepdim:
        out = out.reshape([1 if d in dims else x.shape[d] for d in range(rank)])
    return out


def aten_sum(x: torch.Tensor, dim=None, keepdim: bool = False, *, dtype=None) -> torch.Tensor:
    """aten_functions.py:3311-3346: bool/uint8/int8/int16/int32 promote to int64."""
    if dtype is not None:
        x = x.to(dtype)
    elif not x.dtype.is_floating_point:
        x = x.to(torch.int64)
    dims = _norm_dims(dim, x.dim())
    if x.numel() == 0:  # aten_fast.py:3033-3037: an empty reduction is 0
        shape = [1 if d in dims else s for d, s in enumerate(x.shape)] if keepdim else \
            [s for d, s in enumerate(x.shape) if d not in dims]
        return torch.zeros(shape, dtype=x.dtype)
    return _reduce(x, dims, keepdim, SUM)


def aten_mean(x: torch.Tensor, dim=None, keepdim: bool = False, *, dtype=None) -> torch.Tensor:
    """aten_functions.py:2556-2590 (floating point only, aten_fast.py:2984-3003)."""
    if dtype is not None:
        x = x.to(dtype)
    assert x.dtype in _FLOATS
    return _reduce(x, _norm_dims(dim, x.dim()), keepdim, MEAN)


def aten_amax(x: torch.Tensor, dim=(), keepdim: bool = False) -> torch.Tensor:
    """aten_functions.py:1002-1020: an empty dim list reduces everything."""
    return _reduce(x, _norm_dims(dim, x.dim()), keepdim, AMAX)


def aten_argmax(x: torch.Tensor, dim=None, keepdim: bool = False) -> torch.Tensor:
    """aten_functions.py:1141-1196: ``dim=None`` flattens (keepdim gives an all-ones shape)."""
    if dim is None:
        out = argmax_rows(x.contiguous().reshape(1, -1)).reshape(())
        return out.reshape([1] * x.dim()) if keepdim else out
    dim %= x.dim()
    moved = _move_last(x, dim)
    out = argmax_rows(moved.reshape(-1, moved.shape[-1])).reshape(moved.shape[:-1])
    return out.unsqueeze(dim) if keepdim else out


def aten_mm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """aten_functions.py:2632-2634."""
    return gemm(a, b)


def aten_bmm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """aten_functions.py:1415-1428."""
    return gemm(a, b)


def aten_addmm(inp: torch.Tensor, mat1: torch.Tensor, mat2: torch.Tensor, *, beta=1.0,
               alpha=1.0) -> torch.Tensor:
    """aten_functions.py:971-992. A ``[n]`` input with beta == alpha == 1 takes the fused rule of
    matmul_ops.mojo:2651-2657 (bias added in fp32 before the one cast); every other combination
    is matmul, optional scaling, then a broadcast add, each rounded to the dtype."""
    if beta == 1 and alpha == 1 and inp.dim() == 1 and inp.shape[0] == mat2.shape[1]:
        return gemm(mat1, mat2, inp)
    prod = gemm(mat1, mat2)
    if alpha != 1:
        prod = prod * alpha
    scaled = inp * beta if beta != 1 else inp
    return scaled + prod


def aten_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None):
    """aten_functions.py:2313-2320 with the leading-dim flattening of aten_fast.py:4798-4812."""
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1]) if x.dim() != 2 else x
    out = gemm(x2, weight.t(), bias)
    return out.reshape(*lead, weight.shape[0])


def aten_gelu(x: torch.Tensor, approximate: str = "none") -> torch.Tensor:
    """aten_functions.py:2063-2067."""
    return gelu(x, approximate)
