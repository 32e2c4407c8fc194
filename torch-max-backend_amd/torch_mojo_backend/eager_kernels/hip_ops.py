"""Tensor-level launchers over the C ABI of ``libtmb_hip.so``.

Both surfaces of the backend — the graph registry (``aten_functions``) and the eager
``fast_aten_*`` functions (``aten_fast``) — end up here. Each launcher validates on the host,
allocates its outputs with PyTorch-ROCm's stream-ordered caching allocator (the ownership role
the reference gives to ``TensorHolder``, op_utils/__init__.mojo:250-263), and enqueues the
kernel on the current HIP stream without synchronising.

Inputs must live on a HIP device. CPU tensors are rejected: there is no CPU route.
"""

from __future__ import annotations

import ctypes
import math
import threading
from typing import Optional, Sequence, Tuple

import torch

from torch_mojo_backend import eager_kernels as _ek

_CODES = {
    torch.float32: _ek.F32,
    torch.float16: _ek.F16,
    torch.bfloat16: _ek.BF16,
    torch.int64: _ek.I64,
    torch.int32: _ek.I32,
}
FLOAT_DTYPES = (torch.float32, torch.float16, torch.bfloat16)

_OOM_CODE = 2  # hipErrorOutOfMemory


class HipKernelError(RuntimeError):
    def __init__(self, op: str, code: int):
        self.code = code
        super().__init__(f"{op} failed: {_ek.status_string(code)} (status {code})")


def _check(op: str, code: int) -> None:
    if code == 0:
        return
    if code == _OOM_CODE:
        raise torch.OutOfMemoryError(f"{op}: HIP out of memory")
    raise HipKernelError(op, code)


def require_hip(*tensors: Optional[torch.Tensor]) -> torch.device:
    """All tensors on one HIP device, else TypeError (validated before any allocation)."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if t.device.type != "cuda":
            raise TypeError(
                f"torch_mojo_backend HIP kernels need tensors on a HIP device, got {t.device}; "
                "there is no CPU path"
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise TypeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


_raw_stream = torch._C._cuda_getCurrentRawStream
_current_device = torch.cuda.current_device


def _stream() -> int:
    """The raw hipStream_t of PyTorch's current stream on the current device (the private
    accessor costs a fraction of building a torch.cuda.Stream object per launch)."""
    return _raw_stream(_current_device())


def code_of(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise TypeError(f"dtype {dtype} has no HIP kernel") from None


# ---------------------------------------------------------------------------
# GEMM
# ---------------------------------------------------------------------------
def _matrix_layout(t: torch.Tensor) -> Optional[Tuple[int, int]]:
    """(transposed, leading_dimension) of the last two dims if they are dense row-major or
    dense column-major, else None (same classification as aten_fast.py:4457-4492)."""
    rows, cols = t.shape[-2], t.shape[-1]
    sr, sc = t.stride(-2), t.stride(-1)
    if (sc == 1 or cols == 1) and (sr >= cols or rows == 1):
        return 0, max(sr if rows > 1 else cols, cols, 1)
    if (sr == 1 or rows == 1) and (sc >= rows or cols == 1):
        return 1, max(sc if cols > 1 else rows, rows, 1)
    return None


# Products smaller than this many multiply-adds run as they are: the kernel that takes any layout
# is quick enough there, and re-laying an operand costs launches of its own.
_RELAYOUT_MIN_WORK = 1 << 26


# While a compiled graph without in-place nodes runs, the padded copy of a large operand is kept
# for the next product that pads the same memory to the same width: the gradient of a 50257-wide
# vocabulary projection needs its incoming gradient padded twice, as A of the input gradient and
# as A^T of the weight gradient (0.5 ms per copy at 16384 rows). The entry holds the source tensor,
# so its memory cannot be handed to another tensor while the entry lives; outside such a run the
# dictionary is None and nothing is kept. The dictionary belongs to the thread that runs the graph
# (a backward graph may run on PyTorch's autograd thread while the main thread goes on).
_PAD_STATE = threading.local()
_PAD_REUSE_MIN_BYTES = 64 << 20


def pad_reuse_begin() -> Optional[dict]:
    """Starts keeping padded copies on this thread; returns what `pad_reuse_end` must get back."""
    before = getattr(_PAD_STATE, "reuse", None)
    _PAD_STATE.reuse = {}
    return before


def pad_reuse_end(before: Optional[dict]) -> None:
    _PAD_STATE.reuse = before


def pad_reuse_active() -> Optional[dict]:
    return getattr(_PAD_STATE, "reuse", None)


def _pad_last(x: torch.Tensor, size: int) -> torch.Tensor:
    """`x` with its last dimension zero-padded to `size`, contiguous. Row-major sources go
    through the row-padding kernel (copy speed whatever the source alignment); anything else is
    copied by PyTorch-ROCm's strided copy."""
    reuse, key = getattr(_PAD_STATE, "reuse", None), None
    if reuse is not None and x.numel() * x.element_size() >= _PAD_REUSE_MIN_BYTES:
        key = (x.data_ptr(), tuple(x.shape), x.stride(), x.dtype, size)
        kept = reuse.get(key)
        if kept is not None:
            return kept[1]
    out = _pad_last_copy(x, size)
    if key is not None:
        reuse.clear()
        reuse[key] = (x, out)
    return out


def _pad_last_copy(x: torch.Tensor, size: int) -> torch.Tensor:
    out = torch.empty(tuple(x.shape[:-1]) + (size,), dtype=x.dtype, device=x.device)
    cols = x.shape[-1]
    if out.numel() == 0:
        return out
    flat = x.is_cuda and x.dim() >= 2 and x.stride(-1) == 1 and x.element_size() in (2, 4) and \
        (size * x.element_size()) % 16 == 0 and cols > 0
    if flat:
        # rows must be evenly spaced: [.., rows, cols] with a constant pitch over the leading dims
        pitch = x.stride(-2)
        rows = 1
        for d in range(x.dim() - 2, -1, -1):
            if x.shape[d] != 1 and x.stride(d) != pitch * rows:
                flat = False
                break
            rows *= x.shape[d]
    if flat:
        rc = _ek.lib().tmb_pad_rows(out.data_ptr(), x.data_ptr(), rows, cols, pitch, size,
                                    x.element_size(), _stream())
        if rc == 0:
            return out
        if rc != _ek.ERR_UNSUPPORTED:
            _check("tmb_pad_rows", rc)
    out[..., :cols].copy_(x)
    if size > cols:
        out[..., cols:].zero_()
    return out


def _mfma_layouts_ok(a, b, la, lb, m, n, k, batched, plain_epilogue=True) -> bool:
    """Whether the matrix-core kernels take these operands as they lie (mirrors the library's
    own checks; when it says no, the library would run its any-layout kernel, which is one to two
    orders of magnitude slower on large products)."""
    unit = 16 // a.element_size()  # elements per 16-byte vector: 8 (16-bit) or 4 (fp32)
    if la[1] % unit or lb[1] % unit or a.data_ptr() % 16 or b.data_ptr() % 16:
        return False
    if batched and a.shape[0] > 1 and (a.stride(0) % unit or b.stride(0) % unit):
        return False
    if a.element_size() == 4:
        return (m if la[0] else k) % 4 == 0 and (k if lb[0] else n) % 4 == 0
    if la[0]:  # A stored [K, M]: the weight-gradient form, with B stored [K, N] and no epilogue
        return plain_epilogue and not lb[0] and k % 32 == 0 and k >= 256 and m % 8 == 0 \
            and n % 8 == 0 and n > 64
    return k % 8 == 0


def _relayout_for_mfma(a, b, la, lb, m, n, k, batched, plain=True):
    """Re-lays the operands of a large product so that the matrix-core kernels take it. A
    contraction length or pitch that is not whole 16-byte vectors (a 50257-wide vocabulary as K)
    is zero-padded; B becomes K-major where its own pitch is the obstacle; a transposed A with an
    odd M in the weight-gradient form keeps its form and gets zero columns (the product then has
    a few extra rows, which the caller drops); any other transposed A becomes row-major.
    `plain`: no epilogue and no residual. Returns (a, b, la, lb, k, rows of the launch)."""
    unit = 16 // a.element_size()
    if la[0]:
        b_fits = lb[1] % unit == 0 and b.data_ptr() % 16 == 0
        if a.element_size() == 2:
            keep_form = plain and not batched and b_fits and not lb[0] and k % 32 == 0 \
                and k >= 256 and n % 8 == 0 and n > 64
        else:
            keep_form = not batched and b_fits and (k if lb[0] else n) % 4 == 0
        if keep_form:
            # (the same width as a contraction length of m gets below, so that one padded copy
            # can serve both products of a backward pass)
            mp = m if m % unit == 0 else (m + 63) // 64 * 64
            stored = _pad_last(a.transpose(-1, -2), mp)          # [K, mp], zero columns
            return stored.transpose(-1, -2), b, (1, mp), lb, k, mp
        a = a.contiguous()                      # [.., M, K] row-major (a transposing copy)
    kp = k if k % unit == 0 else (k + 63) // 64 * 64
    if a.shape[-1] != kp or a.stride(-2) % unit or a.data_ptr() % 16 or not a.is_contiguous():
        a = _pad_last(a, kp)
    bt = b.transpose(-1, -2)                    # [.., N, K]
    n_major_ok = not lb[0] and lb[1] % unit == 0 and b.data_ptr() % 16 == 0 and \
        (a.element_size() == 2 or n % 4 == 0)
    k_major_ok = bool(lb[0]) and lb[1] % unit == 0 and b.data_ptr() % 16 == 0 and kp == k
    if n_major_ok:
        if kp != k:                             # rows of zeros below the last k
            grown = torch.empty(tuple(b.shape[:-2]) + (kp, n), dtype=b.dtype, device=b.device)
            grown[..., :k, :].copy_(b)
            grown[..., k:, :].zero_()
            b = grown
    elif not k_major_ok:
        b = _pad_last(bt, kp).transpose(-1, -2)  # K-major, padded along K
    return a, b, _matrix_layout(a), _matrix_layout(b), kp, m


_I64X3 = ctypes.c_int64 * 3
_GEMM_WS_BYTES: dict = {}
_GEMM_PLANS: dict = {}


def gemm_if_planned(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None,
                    epi_flags: int = _ek.EPI_NONE) -> Optional[torch.Tensor]:
    """``gemm(a, b, bias)`` when exactly this operand layout (shapes, strides, dtypes, devices)
    has been validated and launched before, else None: the plan holds the launch arguments, so a
    repeated call (every layer of every decode step) costs one dictionary lookup, one allocation
    and the launch."""
    plan = _GEMM_PLANS.get(
        (a.shape, a.stride(), b.shape, b.stride(), a.dtype, b.dtype, a.device, b.device,
         None if bias is None else (bias.shape, bias.stride(), bias.dtype, bias.device)))
    if plan is None:
        return None
    out_shape, dims, ws_bytes = plan
    out = torch.empty(out_shape, dtype=a.dtype, device=a.device)
    bias_ptr = None if bias is None else bias.data_ptr()
    if ws_bytes:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device)
        rc = _ek.lib().tmb_gemm_ws(out.data_ptr(), a.data_ptr(), b.data_ptr(), bias_ptr,
                                   *dims, epi_flags, ws.data_ptr(), ws_bytes, _stream())
    else:
        rc = _ek.lib().tmb_gemm(out.data_ptr(), a.data_ptr(), b.data_ptr(), bias_ptr,
                                *dims, epi_flags, _stream())
    if rc:
        _check("tmb_gemm", rc)
    return out


def gemm(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None,
         epilogue: int = _ek.EPI_NONE, residual: Optional[torch.Tensor] = None,
         out_dtype: Optional[torch.dtype] = None, round_like_unfused: bool = False) -> torch.Tensor:
    """``epilogue(a @ b + bias) [+ residual]`` for 2-D operands, or 3-D operands with equal batch
    sizes.

    Transposed views (``weight.t()``, ``k.transpose(-2, -1)``) are consumed in place through
    the kernel's transpose flags; other non-dense layouts are materialised once.

    A fused epilogue is evaluated in float32 and cast once: ``T(gelu(acc + bias))``,
    ``T(acc + bias + residual)``. ``round_like_unfused`` instead rounds to the storage type
    wherever a separate kernel would have stored a tensor (the bits of ``gelu(addmm(...))`` and
    of ``addmm(...) + residual``). ``residual`` has the result's shape and the operands' dtype or
    float32; ``out_dtype`` (with a residual only) may be float32 for 16-bit operands: the residual
    stream of a 16-bit model kept in float32.
    """
    epi_flags = epilogue | (_ek.EPI_ROUND_LIKE_UNFUSED if round_like_unfused else 0)
    # Calls that repeat an operand layout already validated (every decode step of a model) go
    # straight to the launch: the key holds everything the checks below look at.
    key = None
    if residual is None and out_dtype is None:
        out = gemm_if_planned(a, b, bias, epi_flags)
        if out is not None:
            return out
        key = True
    a_in, b_in, bias_in = a, b, bias
    require_hip(a, b, bias, residual)
    if a.dtype != b.dtype or a.dtype not in FLOAT_DTYPES:
        raise TypeError(f"gemm: unsupported dtypes {a.dtype} x {b.dtype}")
    batched = a.dim() == 3
    if a.dim() != b.dim() or a.dim() not in (2, 3):
        raise ValueError(f"gemm: expected two 2-D or two 3-D operands, got {a.dim()}-D x {b.dim()}-D")
    if a.shape[-1] != b.shape[-2] or (batched and a.shape[0] != b.shape[0]):
        raise ValueError(f"gemm: shapes {tuple(a.shape)} and {tuple(b.shape)} do not multiply")
    m, k, n = a.shape[-2], a.shape[-1], b.shape[-1]
    batch = a.shape[0] if batched else 1
    if bias is not None:
        if bias.dtype != a.dtype or tuple(bias.shape) != (n,):
            raise ValueError(f"gemm: bias must be [{n}] {a.dtype}, got {tuple(bias.shape)} {bias.dtype}")
        if not bias.is_contiguous():
            bias = bias.contiguous()
    result_dtype = a.dtype if out_dtype is None else out_dtype
    if result_dtype != a.dtype and (result_dtype != torch.float32 or residual is None):
        raise TypeError(f"gemm: {a.dtype} operands cannot produce {result_dtype} "
                        "(float32 results exist together with a residual only)")

    la = _matrix_layout(a)
    if la is None or (batched and batch > 1 and a.stride(0) < 0):
        a = a.contiguous()
        la = (0, max(k, 1))
    lb = _matrix_layout(b)
    if lb is None or (batched and batch > 1 and b.stride(0) < 0):
        b = b.contiguous()
        lb = (0, max(n, 1))
    m_given = m
    if batch * m * n * k >= _RELAYOUT_MIN_WORK and not _mfma_layouts_ok(
            a, b, la, lb, m, n, k, batched, epilogue == _ek.EPI_NONE):
        a, b, la, lb, k, m = _relayout_for_mfma(a, b, la, lb, m, n, k, batched,
                                                epilogue == _ek.EPI_NONE and residual is None)
    out_shape = (batch, m, n) if batched else (m, n)
    if residual is not None and (residual.dtype not in (a.dtype, torch.float32)
                                 or tuple(residual.shape) != out_shape):
        raise ValueError(f"gemm: residual must be {out_shape} {a.dtype} or float32, got "
                         f"{tuple(residual.shape)} {residual.dtype}")
    wide = residual is not None and (residual.dtype != a.dtype or result_dtype != a.dtype)
    if wide and round_like_unfused:
        raise ValueError("gemm: a float32 residual or result keeps the epilogue in float32; "
                         "round_like_unfused does not apply")
    out = torch.empty(out_shape, dtype=result_dtype, device=a.device)
    if out.numel() == 0:
        return out
    lib = _ek.lib()
    # few output tiles and a long K: the library splits K when it is handed scratch memory
    key = (batch, m, n, k, a.dtype)
    ws_bytes = _GEMM_WS_BYTES.get(key)
    if ws_bytes is None:  # a pure function of the shape: asked once per shape
        ws_bytes = _GEMM_WS_BYTES[key] = lib.tmb_gemm_workspace_bytes(batch, m, n, k, code_of(a.dtype))

    def unfused_residual():
        # no kernel carries this epilogue for these operands: product first, then the add.
        # Rounded twice when both live in the storage type, otherwise summed in float32.
        prod = gemm(a, b, bias, epilogue, round_like_unfused=round_like_unfused)
        if wide or not round_like_unfused:
            return (prod.float() + residual.float()).to(result_dtype)
        return prod + residual

    if residual is not None and (ws_bytes or (epilogue != _ek.EPI_NONE and not round_like_unfused)):
        # the split kernels have no residual step; a GELU in front of a float32 add neither
        return unfused_residual()
    if residual is not None:
        res = residual if residual.stride(-1) == 1 and residual.stride(-2) >= n else residual.contiguous()
        rc = lib.tmb_gemm_residual(
            out.data_ptr(), a.data_ptr(), b.data_ptr(), None if bias is None else bias.data_ptr(),
            res.data_ptr(), batch, m, n, k, la[1], lb[1], n, res.stride(-2),
            a.stride(0) if batched else 0, b.stride(0) if batched else 0, m * n,
            res.stride(0) if batched else 0,
            la[0], lb[0], code_of(a.dtype), code_of(res.dtype), code_of(result_dtype), epi_flags,
            _stream())
        if rc == _ek.ERR_UNSUPPORTED:
            return unfused_residual()
        _check("tmb_gemm_residual", rc)
        return out
    if key is not None and a is a_in and b is b_in and bias is bias_in and out_dtype is None:
        # operands are consumed in place: remember the launch arguments for this layout
        if len(_GEMM_PLANS) >= 4096:
            _GEMM_PLANS.clear()
        plan_key = (a.shape, a.stride(), b.shape, b.stride(), a.dtype, b.dtype, a.device, b.device,
                    None if bias is None else (bias.shape, bias.stride(), bias.dtype, bias.device))
        _GEMM_PLANS[plan_key] = (tuple(out.shape),
                                 (batch, m, n, k, la[1], lb[1], n, a.stride(0) if batched else 0,
                                  b.stride(0) if batched else 0, m * n, la[0], lb[0], code_of(a.dtype)),
                                 ws_bytes)
    if ws_bytes:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device)
        rc = lib.tmb_gemm_ws(
            out.data_ptr(), a.data_ptr(), b.data_ptr(), None if bias is None else bias.data_ptr(),
            batch, m, n, k, la[1], lb[1], n, 0, 0, m * n, la[0], lb[0], code_of(a.dtype), epi_flags,
            ws.data_ptr(), ws_bytes, _stream())
        _check("tmb_gemm_ws", rc)
        return out if m == m_given else out[:m_given]  # rows of a padded M are dropped (a view)
    rc = lib.tmb_gemm(
        out.data_ptr(), a.data_ptr(), b.data_ptr(), None if bias is None else bias.data_ptr(),
        batch, m, n, k, la[1], lb[1], n,
        a.stride(0) if batched else 0, b.stride(0) if batched else 0, m * n,
        la[0], lb[0], code_of(a.dtype), epi_flags, _stream())
    _check("tmb_gemm", rc)
    return out if m == m_given else out[:m_given]


# ---------------------------------------------------------------------------
# Row kernels
# ---------------------------------------------------------------------------
def _as_rows(x: torch.Tensor, dim: int) -> Tuple[torch.Tensor, bool]:
    """x with `dim` moved last and made contiguous; flag tells whether a move happened."""
    if dim == x.dim() - 1:
        return (x if x.is_contiguous() else x.contiguous()), False
    return x.movedim(dim, -1).contiguous(), True


def softmax(x: torch.Tensor, dim: int, half_to_float: bool = False, log: bool = False) -> torch.Tensor:
    require_hip(x)
    if x.dtype not in FLOAT_DTYPES:
        raise TypeError(f"softmax: unsupported dtype {x.dtype}")
    out_dtype = torch.float32 if half_to_float else x.dtype
    if x.dim() == 0:
        return torch.full((), 0.0 if log else 1.0, dtype=out_dtype, device=x.device)
    dim %= x.dim()
    rows_t, moved = _as_rows(x, dim)
    cols = rows_t.shape[-1]
    out = torch.empty(rows_t.shape, dtype=out_dtype, device=x.device)
    if out.numel():
        rc = _ek.lib().tmb_softmax_rows(out.data_ptr(), rows_t.data_ptr(), rows_t.numel() // cols,
                                        cols, code_of(x.dtype), code_of(out_dtype), int(log),
                                        _stream())
        _check("tmb_softmax_rows", rc)
    return out.movedim(-1, dim) if moved else out


def softmax_scaled(x: torch.Tensor, scale: float, causal_q_len: int = 0,
                   round_scaled: bool = False) -> torch.Tensor:
    """softmax(x * scale) over the last dimension; with ``causal_q_len`` = q > 0 the tensor is
    read as [..., q, cols] and column j of query row r takes part only if j <= r (the
    reference's ``_softmax_rows(scale, causal, q_len)``, nn_ops.mojo:413-493)."""
    require_hip(x)
    if x.dtype not in FLOAT_DTYPES:
        raise TypeError(f"softmax_scaled: unsupported dtype {x.dtype}")
    if x.dim() < 1:
        raise ValueError("softmax_scaled needs at least one dimension")
    if causal_q_len < 0 or (causal_q_len and (x.dim() < 2 or x.shape[-2] != causal_q_len)):
        raise ValueError(f"softmax_scaled: causal_q_len {causal_q_len} does not match input "
                         f"{tuple(x.shape)}")
    xc = x if x.is_contiguous() else x.contiguous()
    out = torch.empty_like(xc)
    cols = xc.shape[-1]
    if out.numel():
        rc = _ek.lib().tmb_softmax_rows_scaled(out.data_ptr(), xc.data_ptr(), xc.numel() // cols,
                                               cols, code_of(x.dtype), float(scale),
                                               int(bool(round_scaled)), int(causal_q_len), _stream())
        _check("tmb_softmax_rows_scaled", rc)
    return out


def attention_supported(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> bool:
    """True when `attention` can take these [batch, heads, tokens, 64] tensors as they are."""
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        return False
    if q.dtype not in (torch.bfloat16, torch.float16) or k.dtype != q.dtype or v.dtype != q.dtype:
        return False
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        return False
    b, h, t, d = q.shape
    if d != 64 or tuple(k.shape) != (b, h, k.shape[2], 64) or tuple(v.shape) != tuple(k.shape):
        return False
    if k.shape[2] == 0 or b * h * ((t + 127) // 128) >= 1 << 31 or b * h * t == 0:
        return False
    for x in (q, k, v):
        if x.stride(3) != 1 or any(s % 8 or s < 0 for s in x.stride()[:3]) or x.data_ptr() % 16:
            return False
        if (x.shape[2] * x.stride(2) + 64) * 2 >= 1 << 32:
            return False
    return True


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, causal: bool,
              round_like_unfused: bool = False, return_lse: bool = False,
              like_query: bool = False):
    """softmax(scale * q k^T [causal]) v for [batch, heads, tokens, 64] tensors (any strides
    `attention_supported` accepts). Returns a [batch, q_len, heads, 64] contiguous tensor, i.e.
    the layout `y.transpose(1, 2).contiguous()` would have produced; with `like_query` a
    [batch, heads, q_len, 64] tensor laid out as `torch.empty_like(q)` (what ATen's fused attention
    ops return). With `return_lse` also the float32 [batch, heads, q_len] log-sum-exp of every
    query's scores, which `attention_backward` needs."""
    require_hip(q, k, v)
    if not (scale > 0.0 and math.isfinite(scale)):
        raise ValueError(f"attention: scale must be positive and finite, got {scale}")
    if not attention_supported(q, k, v):
        raise ValueError(f"attention: unsupported operands q{tuple(q.shape)} {q.dtype} "
                         f"strides {q.stride()} / k{tuple(k.shape)} / v{tuple(v.shape)}")
    b, h, t, d = q.shape
    i64x3 = ctypes.c_int64 * 3
    strides = [i64x3(x.stride(0), x.stride(1), x.stride(2)) for x in (q, k, v)]
    if like_query:
        out = _gradient_like(q)
        o_str = i64x3(out.stride(0), out.stride(1), out.stride(2))
    else:
        out = torch.empty((b, t, h, d), dtype=q.dtype, device=q.device)
        o_str = i64x3(out.stride(0), out.stride(2), out.stride(1))
    lse = torch.empty((b, h, t), dtype=torch.float32, device=q.device) if return_lse else None
    rc = _ek.lib().tmb_attention_fwd(out.data_ptr(), lse.data_ptr() if return_lse else None,
                                     q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                     b, h, t, k.shape[2], d, strides[0], strides[1], strides[2],
                                     o_str, float(scale), int(bool(causal)),
                                     int(bool(round_like_unfused)), code_of(q.dtype), _stream())
    _check("tmb_attention_fwd", rc)
    return (out, lse) if return_lse else out


def _gradient_like(x: torch.Tensor) -> torch.Tensor:
    """A [batch, heads, tokens, 64] buffer laid out as `torch.empty_like(x)` when the kernels can
    write that layout (rows of 64 contiguous, strides multiples of 4), token-major otherwise."""
    like = torch.empty_like(x)
    if like.stride(3) == 1 and all(s % 4 == 0 and s >= 0 for s in like.stride()[:3]):
        return like
    b, h, t, d = x.shape
    return torch.empty((b, t, h, d), dtype=x.dtype, device=x.device).transpose(1, 2)


def attention_backward_supported(dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor,
                                 v: torch.Tensor, out: torch.Tensor, lse: torch.Tensor) -> bool:
    """True when `attention_backward` takes these tensors as they are: q, k, v as for `attention`,
    `out` and `dout` [batch, heads, q_len, 64] views with the same stride rules, `lse` float32
    [batch, heads, q_len] contiguous."""
    if not attention_supported(q, k, v):
        return False
    b, h, t, d = q.shape
    for x in (out, dout):
        if not x.is_cuda or x.dtype != q.dtype or tuple(x.shape) != (b, h, t, d):
            return False
        if x.stride(3) != 1 or any(s % 8 or s < 0 for s in x.stride()[:3]) or x.data_ptr() % 16:
            return False
    if (t * dout.stride(2) + 64) * 2 >= 1 << 32 or (t * q.stride(2) + 64) * 2 >= 1 << 32:
        return False
    return (lse.is_cuda and lse.dtype == torch.float32 and tuple(lse.shape) == (b, h, t)
            and lse.is_contiguous())


def attention_backward(dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                       out: torch.Tensor, lse: torch.Tensor, scale: float, causal: bool,
                       packed: bool = False, grad_strides=None):
    """(dq, dk, dv) of `attention`: `out` and `dout` are [batch, heads, q_len, 64] views (the
    transposed view of what `attention` returned, and the gradient in the same layout), `lse` what
    `attention(..., return_lse=True)` returned. Each gradient is laid out as
    `torch.empty_like` of its input (what ATen's fused attention backward returns); with `packed`
    and q_len == kv_len the three are [batch, heads, tokens, 64] views of one
    [batch, tokens, 3, heads, 64] buffer, so the gradient of a packed q/k/v projection needs no
    concatenation. `grad_strides`: three stride tuples (or None) for dq, dk, dv where a caller
    needs particular layouts; a layout the kernels cannot write (head_dim not contiguous, strides
    not multiples of 4) is ignored and the default used."""
    require_hip(dout, q, k, v, out, lse)
    if not (scale > 0.0 and math.isfinite(scale)):
        raise ValueError(f"attention_backward: scale must be positive and finite, got {scale}")
    if not attention_backward_supported(dout, q, k, v, out, lse):
        raise ValueError("attention_backward: unsupported operands (see attention_backward_supported)")
    b, h, t, d = q.shape
    s_len = k.shape[2]
    if packed and t == s_len:
        buf = torch.empty((b, t, 3, h, d), dtype=q.dtype, device=q.device)
        dq, dk, dv = (buf[:, :, i].transpose(1, 2) for i in range(3))
    else:
        grads = []
        for x, want in zip((q, k, v), grad_strides or (None, None, None)):
            if want is not None and len(want) == 4 and want[3] == 1 and \
                    all(st % 4 == 0 and st >= 0 for st in want[:3]):
                grads.append(torch.empty_strided(tuple(x.shape), tuple(want), dtype=x.dtype,
                                                 device=x.device))
            else:
                grads.append(_gradient_like(x))
        dq, dk, dv = grads
    lib = _ek.lib()
    workspace = torch.empty(max(int(lib.tmb_attention_bwd_workspace_bytes(b, h, t)), 16),
                            dtype=torch.uint8, device=q.device)
    i64x3 = ctypes.c_int64 * 3
    st = [i64x3(x.stride(0), x.stride(1), x.stride(2)) for x in (q, k, v, out, dout, dq, dk, dv)]
    rc = lib.tmb_attention_bwd(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dout.data_ptr(),
                               q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                               lse.data_ptr(), workspace.data_ptr(), b, h, t, s_len, d, *st,
                               float(scale), int(bool(causal)), code_of(q.dtype), _stream())
    _check("tmb_attention_bwd", rc)
    return dq, dk, dv


# Queries per (batch, head) up to which the decode kernel (one wave per query row, K and V read
# once per query) is used instead of the GEMM-based paths.
DECODE_MAX_QUERIES = 16


def attention_decode_supported(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                               attn_mask: Optional[torch.Tensor]) -> bool:
    """True when `attention_decode` takes these [batch, heads, tokens, head_dim] tensors."""
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4 or not (q.is_cuda and k.is_cuda and v.is_cuda):
        return False
    if q.dtype not in (torch.bfloat16, torch.float16) or k.dtype != q.dtype or v.dtype != q.dtype:
        return False
    b, h, t, d = q.shape
    if d not in (64, 128) or t == 0 or t > DECODE_MAX_QUERIES or k.shape[2] == 0:
        return False
    if tuple(k.shape) != (b, h, k.shape[2], d) or tuple(v.shape) != tuple(k.shape):
        return False
    for x in (q, k, v):
        if x.stride(3) != 1 or any(s % 8 or s < 0 for s in x.stride()[:3]) or x.data_ptr() % 16:
            return False
    if attn_mask is not None:
        if attn_mask.dtype != torch.bool or not attn_mask.is_cuda or attn_mask.dim() > 4:
            return False
        try:
            torch.broadcast_shapes(tuple(attn_mask.shape), (b, h, t, k.shape[2]))
        except RuntimeError:
            return False
        if tuple(torch.broadcast_shapes(tuple(attn_mask.shape), (b, h, t, k.shape[2]))) != (b, h, t, k.shape[2]):
            return False
    return True


def attention_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     causal: bool, attn_mask: Optional[torch.Tensor] = None,
                     checked: bool = False) -> torch.Tensor:
    """softmax(scale q kᵀ [masked]) v for a few queries per head in one launch; returns
    [batch, heads, tokens, head_dim] contiguous. `checked`: the caller has just seen
    `attention_decode_supported` accept exactly these operands."""
    if not checked:
        require_hip(q, k, v, attn_mask)
        if not attention_decode_supported(q, k, v, attn_mask):
            raise ValueError("attention_decode: unsupported operands (see attention_decode_supported)")
    b, h, t, d = q.shape
    out = torch.empty((b, h, t, d), dtype=q.dtype, device=q.device)
    i64x3 = _I64X3
    mask_ptr, mask_strides = None, None
    if attn_mask is not None:
        m4 = attn_mask.expand(b, h, t, k.shape[2])  # stride 0 where it broadcasts
        mask_ptr, mask_strides = m4.data_ptr(), (ctypes.c_int64 * 4)(*m4.stride())
    qs, ks, vs = q.stride(), k.stride(), v.stride()
    rc = _ek.lib().tmb_attention_decode(
        out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), mask_ptr, b, h, t, k.shape[2], d,
        i64x3(qs[0], qs[1], qs[2]), i64x3(ks[0], ks[1], ks[2]), i64x3(vs[0], vs[1], vs[2]),
        i64x3(h * t * d, t * d, d), mask_strides, float(scale), int(bool(causal)),
        _CODES[q.dtype], _stream())
    _check("tmb_attention_decode", rc)
    return out


def attention_composed(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                       causal: bool, attn_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``softmax(q kᵀ · scale + mask) v`` for [..., tokens, head_dim] operands of any head size and
    dtype, built from the GEMM and softmax kernels the way the reference builds it from matmul,
    softmax and matmul graph ops (aten_functions.py:3029-3087). ``attn_mask`` is boolean (True =
    takes part) or additive, broadcastable to the scores; ``causal`` is the top-left aligned
    lower triangle. Returns [..., tokens, head_dim_v]."""
    require_hip(q, k, v, attn_mask)
    if q.dim() < 2 or k.shape[:-2] != q.shape[:-2] or v.shape[:-2] != q.shape[:-2]:
        raise ValueError(f"attention_composed: shapes {tuple(q.shape)}, {tuple(k.shape)}, "
                         f"{tuple(v.shape)} do not match")
    lead = tuple(q.shape[:-2])
    t, s_len = q.shape[-2], k.shape[-2]
    q3 = q.reshape(-1, t, q.shape[-1])
    k3 = k.reshape(-1, s_len, k.shape[-1])
    v3 = v.reshape(-1, s_len, v.shape[-1])
    scores = gemm(q3, k3.transpose(1, 2))                       # [batch, t, s]
    if attn_mask is None and scale > 0.0:
        probs = softmax_scaled(scores, scale, t if causal else 0)
    else:
        scores = (scores * scale).view(*lead, t, s_len)
        if attn_mask is not None and attn_mask.dtype == torch.bool:
            scores = scores.masked_fill(~attn_mask, float("-inf"))
        elif attn_mask is not None:
            scores = scores + attn_mask.to(scores.dtype)
        scores = scores.reshape(-1, t, s_len)
        probs = softmax_scaled(scores, 1.0, t if causal else 0)
    return gemm(probs, v3).view(*lead, t, v.shape[-1])


_LN_PLANS: dict = {}


def layer_norm(x: torch.Tensor, normalized_shape: Sequence[int], weight: Optional[torch.Tensor],
               bias: Optional[torch.Tensor], eps: float, need_stats: bool = True,
               out_dtype: Optional[torch.dtype] = None):
    """(out, mean, rstd); mean/rstd are float32 with shape ``x.shape[:-k] + (1,)*k`` or None
    when ``need_stats`` is False. ``out_dtype`` (default: the input's) may be a 16-bit type for
    a float32 input: the row is read in float32 and the result cast once; weight and bias then
    have the output's type."""
    # a layout already validated (every layer of every decode step): straight to the launch
    key = (x.shape, x.stride(), x.dtype, x.device, tuple(normalized_shape), out_dtype, need_stats,
           None if weight is None else (weight.shape, weight.stride(), weight.dtype, weight.device),
           None if bias is None else (bias.shape, bias.stride(), bias.dtype, bias.device))
    plan = _LN_PLANS.get(key)
    if plan is not None:
        rows, cols, stat_shape, in_code, out_code, odt = plan
        out = torch.empty(x.shape, dtype=odt, device=x.device)
        mean = rstd = None
        if need_stats:
            mean = torch.empty(stat_shape, dtype=torch.float32, device=x.device)
            rstd = torch.empty(stat_shape, dtype=torch.float32, device=x.device)
        rc = _ek.lib().tmb_layer_norm_rows(
            out.data_ptr(), None if mean is None else mean.data_ptr(),
            None if rstd is None else rstd.data_ptr(), x.data_ptr(),
            None if weight is None else weight.data_ptr(), None if bias is None else bias.data_ptr(),
            rows, cols, float(eps), in_code, out_code, _stream())
        _check("tmb_layer_norm_rows", rc)
        return out, mean, rstd
    require_hip(x, weight, bias)
    k = len(normalized_shape)
    out_dtype = x.dtype if out_dtype is None else out_dtype
    if x.dtype not in FLOAT_DTYPES or k < 1 or x.dim() < k or \
            tuple(x.shape[x.dim() - k:]) != tuple(normalized_shape):
        raise ValueError(f"layer_norm: input {tuple(x.shape)} {x.dtype} vs normalized_shape "
                         f"{tuple(normalized_shape)}")
    if out_dtype != x.dtype and not (x.dtype == torch.float32 and out_dtype in FLOAT_DTYPES):
        raise TypeError(f"layer_norm: {x.dtype} input cannot be normalised into {out_dtype}")
    for name, p in (("weight", weight), ("bias", bias)):
        if p is not None and (p.dtype != out_dtype or tuple(p.shape) != tuple(normalized_shape)):
            raise ValueError(f"layer_norm: {name} must be {tuple(normalized_shape)} {out_dtype}")
    cols = math.prod(normalized_shape)
    xc = x if x.is_contiguous() else x.contiguous()
    rows = xc.numel() // cols if cols else 0
    out = torch.empty(xc.shape, dtype=out_dtype, device=x.device)
    stat_shape = tuple(x.shape[: x.dim() - k]) + (1,) * k
    mean = rstd = None
    if need_stats:
        mean = torch.empty(stat_shape, dtype=torch.float32, device=x.device)
        rstd = torch.empty(stat_shape, dtype=torch.float32, device=x.device)
    if xc.numel():
        w = None if weight is None else (weight if weight.is_contiguous() else weight.contiguous())
        b = None if bias is None else (bias if bias.is_contiguous() else bias.contiguous())
        rc = _ek.lib().tmb_layer_norm_rows(
            out.data_ptr(), None if mean is None else mean.data_ptr(),
            None if rstd is None else rstd.data_ptr(), xc.data_ptr(),
            None if w is None else w.data_ptr(), None if b is None else b.data_ptr(),
            rows, cols, float(eps), code_of(x.dtype), code_of(out_dtype), _stream())
        _check("tmb_layer_norm_rows", rc)
        if xc is x and (weight is None or w is weight) and (bias is None or b is bias):
            if len(_LN_PLANS) >= 1024:
                _LN_PLANS.clear()
            _LN_PLANS[key] = (rows, cols, stat_shape, code_of(x.dtype), code_of(out_dtype), out_dtype)
    return out, mean, rstd


def _reduce_geometry(x: torch.Tensor, dims: Sequence[int]):
    """Kept dims (ascending) then reduce dims, made contiguous: the [rows, cols] view of
    op_utils/__init__.mojo:651-720. Returns (rows_tensor, rows, cols, kept_shape)."""
    rank = x.dim()
    dims = list(dims)
    kept = [d for d in range(rank) if d not in dims]
    trailing = dims == list(range(rank - len(dims), rank))
    if trailing and x.is_contiguous():
        moved = x
    else:
        moved = x.permute(kept + dims).contiguous()
    cols = math.prod(x.shape[d] for d in dims)
    rows = math.prod(x.shape[d] for d in kept)
    return moved, rows, cols, [x.shape[d] for d in kept]


def _workspace(rows: int, cols: int, code: int, device, argmax: bool = False) -> Tuple[Optional[torch.Tensor], int]:
    lib = _ek.lib()
    nbytes = (lib.tmb_argmax_workspace_bytes if argmax else lib.tmb_reduce_workspace_bytes)(rows, cols, code)
    if nbytes == 0:
        return None, 0
    return torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes


# Below this many elements the transposing route costs the same few microseconds.
_COLS_KERNEL_MIN_ELEMENTS = 1 << 14


def reduce(x: torch.Tensor, dims: Sequence[int], keepdim: bool, op: int) -> torch.Tensor:
    """sum / mean / amax over `dims` (already normalised, sorted, unique, non-empty unless
    x is 0-d). Output dtype = input dtype."""
    require_hip(x)
    code = code_of(x.dtype)
    rank = x.dim()
    dims = list(dims)
    # The leading dims of a contiguous float tensor (the bias gradient of a linear layer,
    # sum(x, dim=0)): reduced in place by the column kernel instead of transposing first.
    lead = len(dims)
    if 0 < lead < rank and dims == list(range(lead)) and x.dtype in FLOAT_DTYPES \
            and x.is_contiguous() and x.numel() >= _COLS_KERNEL_MIN_ELEMENTS:
        n_rows = math.prod(x.shape[:lead])
        n_cols = math.prod(x.shape[lead:])
        if 0 < n_rows < (1 << 40) and n_cols > 0:
            lib = _ek.lib()
            out = torch.empty(tuple(x.shape[lead:]), dtype=x.dtype, device=x.device)
            nbytes = int(lib.tmb_reduce_cols_workspace_bytes(n_rows, n_cols, code))
            ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
            rc = lib.tmb_reduce_cols(out.data_ptr(), x.data_ptr(), n_rows, n_cols, op, code,
                                     ws.data_ptr(), nbytes, _stream())
            if rc != _ek.ERR_UNSUPPORTED:
                _check("tmb_reduce_cols", rc)
                return out.reshape([1] * lead + list(x.shape[lead:])) if keepdim else out
    moved, rows, cols, kept_shape = _reduce_geometry(x, dims)
    if cols == 0 or rows == 0:
        raise ValueError("reduce: empty reduction has no kernel; the caller decides its value")
    out = torch.empty(kept_shape, dtype=x.dtype, device=x.device)
    ws, ws_bytes = _workspace(rows, cols, code, x.device)
    rc = _ek.lib().tmb_reduce_rows(out.data_ptr(), moved.data_ptr(), rows, cols, op, code,
                                   None if ws is None else ws.data_ptr(), ws_bytes, _stream())
    _check("tmb_reduce_rows", rc)
    if keepdim:
        out = out.reshape([1 if d in dims else x.shape[d] for d in range(rank)])
    return out


def argmax(x: torch.Tensor, dim: Optional[int], keepdim: bool) -> torch.Tensor:
    require_hip(x)
    code = code_of(x.dtype)
    if x.numel() == 0:
        raise ValueError("argmax of an empty tensor")
    rank = x.dim()
    if dim is None:
        dims = list(range(rank))
    else:
        dims = [dim % rank] if rank else []
    moved, rows, cols, kept_shape = _reduce_geometry(x, dims)
    out = torch.empty(kept_shape, dtype=torch.int64, device=x.device)
    ws, ws_bytes = _workspace(rows, cols, code, x.device, argmax=True)
    rc = _ek.lib().tmb_argmax_rows(out.data_ptr(), moved.data_ptr(), rows, cols, code,
                                   None if ws is None else ws.data_ptr(), ws_bytes, _stream())
    _check("tmb_argmax_rows", rc)
    if keepdim:
        out = out.reshape([1 if d in dims else x.shape[d] for d in range(rank)])
    return out


def embedding(table: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """``table[indices]`` for a 2-D float table and int32 / int64 indices of any shape
    (reference: aten_fast.py:5336-5371). Indices outside the table read the nearest valid row."""
    require_hip(table, indices)
    if table.dim() != 2 or table.dtype not in FLOAT_DTYPES:
        raise TypeError(f"embedding: table must be a 2-D float tensor, got {tuple(table.shape)} {table.dtype}")
    if indices.dtype not in (torch.int64, torch.int32):
        raise TypeError(f"embedding: indices must be int32 or int64, got {indices.dtype}")
    rows, row_len = table.shape
    out = torch.empty(tuple(indices.shape) + (row_len,), dtype=table.dtype, device=table.device)
    if out.numel() == 0:
        return out
    if rows == 0:
        raise IndexError("embedding: lookup in an empty table")
    t = table if table.is_contiguous() else table.contiguous()
    i = indices if indices.is_contiguous() else indices.contiguous()
    rc = _ek.lib().tmb_gather_rows(out.data_ptr(), t.data_ptr(), i.data_ptr(), i.numel(), row_len,
                                   rows, code_of(table.dtype),
                                   _ek.I64 if indices.dtype == torch.int64 else _ek.I32, _stream())
    _check("tmb_gather_rows", rc)
    return out


def cat2_supported(a: torch.Tensor, b: torch.Tensor, dim: int) -> bool:
    """True when `cat2` takes these two tensors: same device, dtype and rank, equal sizes apart
    from `dim` (already normalised), both contiguous, not both empty."""
    if a.dtype != b.dtype or a.device != b.device or not a.is_cuda or a.dim() != b.dim() \
            or not 0 <= dim < a.dim() or not (a.is_contiguous() and b.is_contiguous()):
        return False
    sa, sb = a.shape, b.shape
    for i in range(a.dim()):
        if i != dim and sa[i] != sb[i]:
            return False
    return a.numel() + b.numel() > 0


def cat2(a: torch.Tensor, b: torch.Tensor, dim: int, checked: bool = False) -> torch.Tensor:
    """``torch.cat([a, b], dim)`` for two contiguous tensors in one launch (reference:
    aten_fast.py:2203-2228, the key/value-cache append of a decode step). `checked`: the caller
    has just seen `cat2_supported` accept exactly these operands."""
    if not checked and not cat2_supported(a, b, dim):
        raise ValueError(f"cat2: unsupported operands {tuple(a.shape)} {a.dtype} / "
                         f"{tuple(b.shape)} {b.dtype}, dim {dim}")
    shape = list(a.shape)
    shape[dim] += b.shape[dim]
    out = torch.empty(shape, dtype=a.dtype, device=a.device)
    rows = math.prod(shape[:dim])
    inner = math.prod(shape[dim + 1:]) * a.element_size()
    rc = _ek.lib().tmb_cat2_rows(out.data_ptr(), a.data_ptr(), b.data_ptr(), rows,
                                 a.shape[dim] * inner, b.shape[dim] * inner, _stream())
    _check("tmb_cat2_rows", rc)
    return out


def gelu(x: torch.Tensor, approximate: str = "none") -> torch.Tensor:
    require_hip(x)
    if x.dtype not in FLOAT_DTYPES:
        raise TypeError(f"gelu: unsupported dtype {x.dtype}")
    if approximate not in ("none", "tanh"):
        raise ValueError(f"gelu: approximate must be 'none' or 'tanh', got {approximate!r}")
    xc = x if x.is_contiguous() else x.contiguous()
    out = torch.empty_like(xc)
    if xc.numel():
        rc = _ek.lib().tmb_gelu(out.data_ptr(), xc.data_ptr(), xc.numel(), code_of(x.dtype),
                                int(approximate == "tanh"), _stream())
        _check("tmb_gelu", rc)
    return out


# ---------------------------------------------------------------------------
# Backward twins
# ---------------------------------------------------------------------------
def gelu_backward(grad: torch.Tensor, x: torch.Tensor, approximate: str = "none") -> torch.Tensor:
    """``grad * gelu'(x)`` (reference: activation_backward_ops.mojo:50-73)."""
    require_hip(grad, x)
    if approximate not in ("none", "tanh"):
        raise ValueError(f"gelu_backward: approximate must be 'none' or 'tanh', got {approximate!r}")
    if x.dtype not in FLOAT_DTYPES or grad.dtype != x.dtype or grad.shape != x.shape:
        raise TypeError(f"gelu_backward: {tuple(grad.shape)} {grad.dtype} vs {tuple(x.shape)} {x.dtype}")
    gc = grad if grad.is_contiguous() else grad.contiguous()
    xc = x if x.is_contiguous() else x.contiguous()
    out = torch.empty_like(xc)
    if out.numel():
        _check("tmb_gelu_backward", _ek.lib().tmb_gelu_backward(
            out.data_ptr(), gc.data_ptr(), xc.data_ptr(), out.numel(), code_of(x.dtype),
            int(approximate == "tanh"), _stream()))
    return out


def softmax_backward(grad: torch.Tensor, out: torch.Tensor, dim: int, log: bool) -> torch.Tensor:
    """Gradient of softmax (``log`` False) or log-softmax (True) along ``dim`` from the saved
    output (reference: aten_functions.py:788-833)."""
    require_hip(grad, out)
    if out.dtype not in FLOAT_DTYPES or grad.dtype != out.dtype or grad.shape != out.shape:
        raise TypeError(f"softmax_backward: {tuple(grad.shape)} {grad.dtype} vs "
                        f"{tuple(out.shape)} {out.dtype}")
    if out.dim() == 0:
        return torch.zeros_like(out) if not log else grad - torch.exp(out) * grad
    dim %= out.dim()
    last = out.dim() - 1
    g = grad if dim == last else grad.transpose(dim, last)
    o = out if dim == last else out.transpose(dim, last)
    gc, oc = g.contiguous(), o.contiguous()
    res = torch.empty_like(oc)
    cols = oc.shape[-1]
    if res.numel():
        _check("tmb_softmax_backward_rows", _ek.lib().tmb_softmax_backward_rows(
            res.data_ptr(), gc.data_ptr(), oc.data_ptr(), oc.numel() // cols, cols,
            code_of(out.dtype), int(bool(log)), _stream()))
    return res if dim == last else res.transpose(dim, last).contiguous()


def nll_log_softmax_backward(grad_output: torch.Tensor, logp: torch.Tensor, target: torch.Tensor,
                             total_weight: Optional[torch.Tensor], reduction: int,
                             ignore_index: int) -> torch.Tensor:
    """``_log_softmax_backward_data(nll_loss_backward(grad_output, logp, target, None, reduction,
    ignore_index, total_weight), logp, 1, logp.dtype)`` in one pass over the saved
    log-probabilities ``logp`` [rows, classes], without the dense NLL gradient in between
    (reference: eager_kernels/aten_fast.py:3450-3497 + aten_functions.py:788-833). The result is a
    [rows, classes] view of rows of whole 16-byte vectors with zeros behind each row; while a
    compiled graph keeps padded copies (`pad_reuse_begin`), the products that take it as an
    operand find that buffer instead of padding the view again."""
    require_hip(grad_output, logp, target, total_weight)
    if logp.dim() != 2 or logp.dtype not in FLOAT_DTYPES or target.dtype != torch.int64 or \
            tuple(target.shape) != (logp.shape[0],) or reduction not in (0, 1, 2):
        raise TypeError(f"nll_log_softmax_backward: logp {tuple(logp.shape)} {logp.dtype}, target "
                        f"{tuple(target.shape)} {target.dtype}, reduction {reduction}")
    rows, cols = logp.shape
    if grad_output.numel() != (rows if reduction == 0 else 1) or \
            (reduction == 1 and (total_weight is None or total_weight.numel() != 1)):
        raise ValueError("nll_log_softmax_backward: grad_output / total_weight do not fit the reduction")
    lp = logp if logp.stride(1) == 1 and (rows <= 1 or logp.stride(0) >= cols) else logp.contiguous()
    go = grad_output.to(logp.dtype).contiguous()
    tw = None if total_weight is None else total_weight.to(logp.dtype).contiguous()
    unit = 16 // logp.element_size()
    ldo = cols if cols % unit == 0 else (cols + 63) // 64 * 64   # the width `_relayout_for_mfma` pads to
    buf = torch.empty((rows, ldo), dtype=logp.dtype, device=logp.device)
    if buf.numel():
        _check("tmb_nll_log_softmax_backward_rows", _ek.lib().tmb_nll_log_softmax_backward_rows(
            buf.data_ptr(), lp.data_ptr(), target.contiguous().data_ptr(), go.data_ptr(),
            None if tw is None else tw.data_ptr(), rows, cols, lp.stride(0) if rows > 1 else cols, ldo,
            int(reduction), int(ignore_index), code_of(logp.dtype), _stream()))
    if ldo == cols:
        return buf
    out = buf[:, :cols]
    reuse = getattr(_PAD_STATE, "reuse", None)
    if reuse is not None and out.numel() * out.element_size() >= _PAD_REUSE_MIN_BYTES:
        reuse.clear()
        reuse[(out.data_ptr(), tuple(out.shape), out.stride(), out.dtype, ldo)] = (out, buf)
    return out


def layer_norm_backward(grad: torch.Tensor, x: torch.Tensor, normalized_shape: Sequence[int],
                        mean: torch.Tensor, rstd: torch.Tensor, weight: Optional[torch.Tensor],
                        output_mask: Sequence[bool]):
    """(grad_input, grad_weight, grad_bias), each None where ``output_mask`` says so
    (reference: aten_fast.py:2797-2913). ``mean`` / ``rstd`` are the float32 statistics the
    forward returned."""
    require_hip(grad, x, mean, rstd, weight)
    normalized_shape = tuple(normalized_shape)
    k = len(normalized_shape)
    if x.dtype not in FLOAT_DTYPES or grad.dtype != x.dtype or grad.shape != x.shape or k < 1 \
            or tuple(x.shape[x.dim() - k:]) != normalized_shape:
        raise ValueError(f"layer_norm_backward: grad {tuple(grad.shape)} {grad.dtype}, input "
                         f"{tuple(x.shape)} {x.dtype}, normalized_shape {normalized_shape}")
    cols = math.prod(normalized_shape)
    rows = x.numel() // cols if cols else 0
    if mean.dtype != torch.float32 or rstd.dtype != torch.float32 or mean.numel() != rows \
            or rstd.numel() != rows:
        raise ValueError("layer_norm_backward: mean / rstd must be float32 with one value per row")
    if weight is not None and (weight.dtype != x.dtype or tuple(weight.shape) != normalized_shape):
        raise ValueError(f"layer_norm_backward: weight must be {normalized_shape} {x.dtype}")
    want_x, want_w, want_b = (bool(m) for m in output_mask)
    gc, xc = grad.contiguous(), x.contiguous()
    dx = torch.empty_like(xc) if want_x else None
    dw = torch.empty(normalized_shape, dtype=x.dtype, device=x.device) if want_w else None
    db = torch.empty(normalized_shape, dtype=x.dtype, device=x.device) if want_b else None
    if rows == 0 or cols == 0:
        for t in (dw, db):
            if t is not None:
                t.zero_()
        return dx, dw, db
    code = code_of(x.dtype)
    ws, ws_bytes = None, 0
    if want_w or want_b:
        ws_bytes = _ek.lib().tmb_layer_norm_backward_workspace_bytes(rows, cols, code)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    wc = None if weight is None else weight.contiguous()
    _check("tmb_layer_norm_backward_rows", _ek.lib().tmb_layer_norm_backward_rows(
        None if dx is None else dx.data_ptr(), None if dw is None else dw.data_ptr(),
        None if db is None else db.data_ptr(), gc.data_ptr(), xc.data_ptr(),
        mean.contiguous().data_ptr(), rstd.contiguous().data_ptr(),
        None if wc is None else wc.data_ptr(), rows, cols, code,
        None if ws is None else ws.data_ptr(), ws_bytes, _stream()))
    return dx, dw, db


def layer_norm_backward_add(grad: torch.Tensor, x: torch.Tensor, normalized_shape: Sequence[int],
                            mean: torch.Tensor, rstd: torch.Tensor, weight: Optional[torch.Tensor],
                            addend: Optional[torch.Tensor], want_sum: bool):
    """``layer_norm_backward`` with all three outputs where its grad_input re-joins a residual
    stream: returns (grad_input + addend, grad_weight, grad_bias, column sums of the first over
    all leading dimensions or None), each stored in the tensor type step by step as the separate
    ops would (this one, ``aten.add``, ``aten.sum``). Returns None when the shape is outside the
    one-pass kernels: the caller then runs the separate ops."""
    require_hip(grad, x, mean, rstd, weight, addend)
    normalized_shape = tuple(normalized_shape)
    k = len(normalized_shape)
    if addend is None and not want_sum:
        raise ValueError("layer_norm_backward_add: neither an addend nor the column sums are asked for")
    if x.dtype not in FLOAT_DTYPES or grad.dtype != x.dtype or grad.shape != x.shape or k < 1 \
            or tuple(x.shape[x.dim() - k:]) != normalized_shape:
        raise ValueError(f"layer_norm_backward_add: grad {tuple(grad.shape)} {grad.dtype}, input "
                         f"{tuple(x.shape)} {x.dtype}, normalized_shape {normalized_shape}")
    if addend is not None and (addend.dtype != x.dtype or addend.shape != x.shape):
        raise ValueError(f"layer_norm_backward_add: addend {tuple(addend.shape)} {addend.dtype} for "
                         f"input {tuple(x.shape)} {x.dtype}")
    cols = math.prod(normalized_shape)
    rows = x.numel() // cols if cols else 0
    if mean.dtype != torch.float32 or rstd.dtype != torch.float32 or mean.numel() != rows \
            or rstd.numel() != rows:
        raise ValueError("layer_norm_backward_add: mean / rstd must be float32 with one value per row")
    if weight is not None and (weight.dtype != x.dtype or tuple(weight.shape) != normalized_shape):
        raise ValueError(f"layer_norm_backward_add: weight must be {normalized_shape} {x.dtype}")
    if rows == 0 or cols == 0:
        return None
    code = code_of(x.dtype)
    lib = _ek.lib()
    ws_bytes = int(lib.tmb_layer_norm_backward_add_workspace_bytes(rows, cols, code))
    if ws_bytes == 0:
        return None
    gc, xc = grad.contiguous(), x.contiguous()
    ac = None if addend is None else addend.contiguous()
    wc = None if weight is None else weight.contiguous()
    dx = torch.empty_like(xc)
    dw = torch.empty(normalized_shape, dtype=x.dtype, device=x.device)
    db = torch.empty(normalized_shape, dtype=x.dtype, device=x.device)
    ds = torch.empty(normalized_shape, dtype=x.dtype, device=x.device) if want_sum else None
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    rc = lib.tmb_layer_norm_backward_add_rows(
        dx.data_ptr(), dw.data_ptr(), db.data_ptr(), None if ds is None else ds.data_ptr(),
        gc.data_ptr(), xc.data_ptr(), mean.contiguous().data_ptr(), rstd.contiguous().data_ptr(),
        None if wc is None else wc.data_ptr(), None if ac is None else ac.data_ptr(), rows, cols,
        code, ws.data_ptr(), ws_bytes, _stream())
    if rc == _ek.ERR_UNSUPPORTED:
        return None
    _check("tmb_layer_norm_backward_add_rows", rc)
    return dx, dw, db, ds


def linear_backward(x: torch.Tensor, grad: torch.Tensor, weight: torch.Tensor,
                    output_mask: Sequence[bool]):
    """(grad_input, grad_weight, grad_bias) of ``x @ weight.T + bias`` (reference:
    aten_functions.py:2323-2375): grad_input = dy W, grad_weight = dyᵀ x (the transposed-A GEMM),
    grad_bias = column sums of dy. The two parameter outputs are both defined whenever either is
    asked for, as in the reference."""
    require_hip(x, grad, weight)
    if weight.dim() != 2 or x.dim() < 1 or x.shape[-1] != weight.shape[1] \
            or grad.shape[-1] != weight.shape[0] or grad.shape[:-1] != x.shape[:-1]:
        raise ValueError(f"linear_backward: input {tuple(x.shape)}, grad {tuple(grad.shape)}, "
                         f"weight {tuple(weight.shape)}")
    want_x, want_w, want_b = (bool(m) for m in output_mask)
    out_f, in_f = weight.shape
    rows = x.numel() // in_f if in_f else 0
    x2 = x.reshape(rows, in_f)
    g2 = grad.reshape(rows, out_f)
    dx = dw = db = None
    if want_x:
        dx = (torch.zeros_like(x) if out_f == 0 else gemm(g2, weight).view(x.shape))
    if want_w or want_b:
        dw = (torch.zeros_like(weight) if rows == 0 else gemm(g2.t(), x2))
        if want_b and rows > 0:
            db = reduce(g2, [0], False, _ek.SUM)
        else:
            db = torch.zeros(out_f, dtype=grad.dtype, device=grad.device)
    return dx, dw, db


def copy_bytes(dst: torch.Tensor, src: torch.Tensor) -> None:
    """Plain device copy through the library's yardstick kernel (benchmarks only)."""
    require_hip(dst, src)
    nbytes = src.numel() * src.element_size()
    assert dst.numel() * dst.element_size() == nbytes and dst.is_contiguous() and src.is_contiguous()
    _check("tmb_copy_bytes", _ek.lib().tmb_copy_bytes(dst.data_ptr(), src.data_ptr(), nbytes, _stream()))
