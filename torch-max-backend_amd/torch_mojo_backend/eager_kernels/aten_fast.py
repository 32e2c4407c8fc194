"""ATen-signature eager implementations of the hot ops over ``TorchMojoTensor``.

Counterpart of the reference's ``torch_mojo_backend/eager_kernels/aten_fast.py`` for the hot
path. Each ``fast_aten_*`` takes the ATen schema's arguments, validates metadata *before*
allocating or materialising anything (reference :2741-2742), and returns a tensor (or tuple)
or the ``NOT_HANDLED`` sentinel (reference :46) — which the dispatcher turns into a
``NotImplementedError`` naming the op (mojo_device_aten_ops.py:94-119). Supported cases launch
the gfx950 kernels through ``hip_ops``; there is no other route.
"""

from __future__ import annotations

import functools
import math

import torch

import torch_mojo_backend.is_running_tests
from torch_mojo_backend import eager_kernels as _ek
from torch_mojo_backend.eager_kernels import hip_ops
from torch_mojo_backend.mojo_device.torch_mojo_tensor import TorchMojoTensor

NOT_HANDLED = object()

_FLOAT_DTYPES = (torch.float32, torch.float16, torch.bfloat16)
_ROW_REDUCE_DTYPES = _FLOAT_DTYPES + (torch.int64, torch.int32)
_CAST_DTYPES = _FLOAT_DTYPES + (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8,
                                torch.bool)


def _t(x):
    """The mojo tensor behind ``x`` or None."""
    return x if isinstance(x, TorchMojoTensor) else None


_wrap = TorchMojoTensor._adopt  # results of the kernels below: HIP tensors, never part of a graph


def fast_filled(shape, value, dtype, device) -> TorchMojoTensor:
    return _wrap(torch.full(tuple(shape), value, dtype=dtype, device=device))


def _same_device(*tensors) -> bool:
    devs = {t._device for t in tensors if t is not None}
    return len(devs) <= 1


# ---------------------------------------------------------------------------
# Matmul family (reference :4853-5059)
# ---------------------------------------------------------------------------
def _gemm_operands_ok(a, b, rank) -> bool:
    return (a is not None and b is not None and len(a._shape) == rank and len(b._shape) == rank
            and a._dtype == b._dtype and a._dtype in _FLOAT_DTYPES and _same_device(a, b)
            and a._shape[-1] == b._shape[-2])


def fast_aten_mm(x, y):
    a, b = _t(x), _t(y)
    if not _gemm_operands_ok(a, b, 2):
        return NOT_HANDLED
    return _wrap(hip_ops.gemm(a._holder, b._holder))


def fast_aten_addmm(input, mat1, mat2, *, beta=1.0, alpha=1.0):
    # beta/alpha scaling is not implemented by the fast path (reference :4864-4876).
    if beta != 1 or alpha != 1:
        return NOT_HANDLED
    bias, a, b = _t(input), _t(mat1), _t(mat2)
    if bias is not None and a is not None and b is not None:
        # the layout of a previous call (same module, next decode step): checked then
        out = hip_ops.gemm_if_planned(a._holder, b._holder, bias._holder)
        if out is not None:
            return _wrap(out)
    if bias is None or not _gemm_operands_ok(a, b, 2) or not _same_device(a, bias):
        return NOT_HANDLED
    n = b._shape[1]
    if bias._dtype != a._dtype:
        return NOT_HANDLED
    if tuple(bias._shape) == (n,):
        return _wrap(hip_ops.gemm(a._holder, b._holder, bias._holder))
    if tuple(bias._shape) in ((a._shape[0], n), (1, n)):
        # full-matrix input: matmul, then the broadcast add (two roundings, as ATen does)
        prod = hip_ops.gemm(a._holder, b._holder)
        return _wrap(bias._holder + prod)
    return NOT_HANDLED


def fast_aten_linear(input, weight, bias=None):
    """``input @ weight.T + bias``; the weight is read K-major in place, leading dims of the
    input are flattened as a zero-copy view (reference :4798-4812, :4879-4936)."""
    a, w = _t(input), _t(weight)
    bs = _t(bias) if bias is not None else None
    if a is None or w is None or (bias is not None and bs is None):
        return NOT_HANDLED
    if len(w._shape) != 2 or len(a._shape) < 1 or a._shape[-1] != w._shape[1]:
        return NOT_HANDLED
    if a._dtype != w._dtype or a._dtype not in _FLOAT_DTYPES or not _same_device(a, w, bs):
        return NOT_HANDLED
    out_features = w._shape[0]
    if bs is not None and (tuple(bs._shape) != (out_features,) or bs._dtype != a._dtype):
        return NOT_HANDLED
    lead = tuple(a._shape[:-1])
    k = a._shape[-1]
    rows = math.prod(lead)
    if out_features == 0 or rows == 0:
        return _wrap(torch.empty(lead + (out_features,), dtype=a._dtype, device=a._device))
    if k == 0:  # reference :4923-4928
        if bs is not None:
            return _wrap(bs._holder.expand(lead + (out_features,)).clone())
        return fast_filled(lead + (out_features,), 0.0, a._dtype, a._device)
    x2 = a._holder.reshape(rows, k)
    out = hip_ops.gemm(x2, w._holder.t(), None if bs is None else bs._holder)
    return _wrap(out.view(lead + (out_features,)))


def fast_aten_bmm(input, mat2):
    a, b = _t(input), _t(mat2)
    if not _gemm_operands_ok(a, b, 3) or a._shape[0] != b._shape[0]:
        return NOT_HANDLED
    return _wrap(hip_ops.gemm(a._holder, b._holder))


def _fast_aten_bmm_transpose_b(input, mat2):
    """``input @ mat2.transpose(-2, -1)`` without a transpose copy (reference :5045-5059)."""
    a, b = _t(input), _t(mat2)
    if a is None or b is None or len(b._shape) != 3:
        return NOT_HANDLED
    return fast_aten_bmm(a, _wrap(b._holder.transpose(-2, -1)))


# ---------------------------------------------------------------------------
# Softmax family (reference :5294-5328, :3201-3234)
# ---------------------------------------------------------------------------
def fast_aten__softmax(input, dim, half_to_float=False):
    t = _t(input)
    if t is None or t._numel == 0 or t._dtype not in _FLOAT_DTYPES or not isinstance(dim, int) \
            or isinstance(dim, bool):
        return NOT_HANDLED
    if half_to_float and t._dtype not in (torch.float16, torch.bfloat16):
        return NOT_HANDLED
    rank = len(t._shape)
    if rank == 0:
        return fast_filled((), 1.0, torch.float32 if half_to_float else t._dtype, t._device)
    if not -rank <= dim < rank:
        return NOT_HANDLED
    return _wrap(hip_ops.softmax(t._holder, dim % rank, half_to_float=bool(half_to_float)))


def fast_aten_softmax(input, dim=-1, dtype=None):
    if dtype is not None:
        return NOT_HANDLED
    return fast_aten__softmax(input, dim, False)


def fast_aten__log_softmax(input, dim, half_to_float=False):
    t = _t(input)
    if t is None or t._numel == 0 or t._dtype not in _FLOAT_DTYPES or not isinstance(dim, int) \
            or isinstance(dim, bool):
        return NOT_HANDLED
    if half_to_float and t._dtype != torch.float16:  # fp16 only (reference :3213)
        return NOT_HANDLED
    rank = len(t._shape)
    if rank == 0:
        if dim not in (-1, 0):
            return NOT_HANDLED
        return fast_filled((), 0.0, torch.float32 if half_to_float else t._dtype, t._device)
    if not -rank <= dim < rank:
        return NOT_HANDLED
    return _wrap(hip_ops.softmax(t._holder, dim % rank, half_to_float=bool(half_to_float), log=True))


# ---------------------------------------------------------------------------
# Attention (reference :5177-5285)
# ---------------------------------------------------------------------------
def fast_aten_scaled_dot_product_attention(query, key, value, attn_mask=None, dropout_p=0.0,
                                           is_causal=False, *, scale=None, enable_gqa=False):
    q, k, v = _t(query), _t(key), _t(value)
    if q is None or k is None or v is None:
        return NOT_HANDLED
    hq, hk, hv = q._holder, k._holder, v._holder
    # a decode step first (a few queries per head, every layer of every generated token): its
    # own support check covers dtypes, shapes and layouts, so the general checks below are skipped
    if dropout_p == 0.0 and not enable_gqa and hq.dim() == 4 \
            and hq.shape[2] <= hip_ops.DECODE_MAX_QUERIES and hk.device == hq.device \
            and hv.device == hq.device and not (attn_mask is not None and is_causal):
        mask0 = None if attn_mask is None else _t(attn_mask)
        if (attn_mask is None or (mask0 is not None and mask0._holder.device == hq.device)) \
                and hip_ops.attention_decode_supported(hq, hk, hv, None if mask0 is None else mask0._holder):
            s0 = float(scale) if scale is not None else 1.0 / math.sqrt(hq.shape[-1])
            return _wrap(hip_ops.attention_decode(hq, hk, hv, s0, bool(is_causal),
                                                  None if mask0 is None else mask0._holder,
                                                  checked=True))
    if not _same_device(q, k, v):
        return NOT_HANDLED
    if dropout_p != 0.0 or enable_gqa or len(q._shape) < 2 or q._dtype not in _FLOAT_DTYPES \
            or k._dtype != q._dtype or v._dtype != q._dtype:
        return NOT_HANDLED
    if tuple(k._shape[:-2]) != tuple(q._shape[:-2]) or tuple(v._shape[:-2]) != tuple(q._shape[:-2]) \
            or k._shape[-1] != q._shape[-1] or v._shape[-2] != k._shape[-2] or q._numel == 0 \
            or k._shape[-2] == 0:
        return NOT_HANDLED
    mask = None
    if attn_mask is not None:
        mask = _t(attn_mask)
        if mask is None or not _same_device(q, mask) or is_causal:
            return NOT_HANDLED
    s = float(scale) if scale is not None else 1.0 / math.sqrt(q._shape[-1])
    # a few queries per head (a decode step): the memory-bound kernel that reads K and V once,
    # before the 128-query MFMA kernel gets to run tiles with 1-16 live rows
    mask_h = None if mask is None else mask._holder
    if len(q._shape) == 4 and q._shape[2] <= hip_ops.DECODE_MAX_QUERIES \
            and hip_ops.attention_decode_supported(q._holder, k._holder, v._holder, mask_h):
        return _wrap(hip_ops.attention_decode(q._holder, k._holder, v._holder, s, bool(is_causal),
                                              mask_h, checked=True))
    if mask is None and s > 0.0 and len(q._shape) == 4 \
            and hip_ops.attention_supported(q._holder, k._holder, v._holder):
        out = hip_ops.attention(q._holder, k._holder, v._holder, s, bool(is_causal))
        return _wrap(out.transpose(1, 2))  # [batch, heads, tokens, head_dim] view, as ATen returns it
    # other head sizes, fp32, additive masks: GEMM + softmax + GEMM
    return _wrap(hip_ops.attention_composed(q._holder, k._holder, v._holder, s, bool(is_causal),
                                            None if mask is None else mask._holder))


# ---------------------------------------------------------------------------
# Concatenation of two contiguous tensors (reference :2173-2256): the key/value-cache append
# ---------------------------------------------------------------------------
def fast_aten_cat(tensors, dim=0):
    """Two contiguous mojo tensors: one launch of the row-append kernel. Anything else (more
    inputs, strided inputs, the legacy 1-D empty tensor PyTorch skips) is PyTorch-ROCm's cat on
    the holders, as the other cold ops run."""
    if len(tensors) == 2 and type(dim) is int:
        a, b = _t(tensors[0]), _t(tensors[1])
        if a is not None and b is not None:
            ha, hb = a._holder, b._holder
            rank = ha.dim()
            if rank and -rank <= dim < rank and hip_ops.cat2_supported(ha, hb, dim % rank):
                return _wrap(hip_ops.cat2(ha, hb, dim % rank, checked=True))
    holders = []
    for x in tensors:
        t = _t(x)
        if t is None:
            return NOT_HANDLED
        holders.append(t._holder)
    return _wrap(torch.cat(holders, dim))


def _flash_operands(query, key, value, dropout_p, scale):
    """(q, k, v, scale) when the fused kernels take the call, else None."""
    q, k, v = _t(query), _t(key), _t(value)
    if q is None or k is None or v is None or not _same_device(q, k, v) or dropout_p != 0.0 \
            or len(q._shape) != 4:
        return None
    s = float(scale) if scale is not None else 1.0 / math.sqrt(q._shape[-1])
    if not (s > 0.0) or not hip_ops.attention_supported(q._holder, k._holder, v._holder):
        return None
    return q, k, v, s


def fast_aten__scaled_dot_product_flash_attention(query, key, value, dropout_p=0.0,
                                                  is_causal=False, return_debug_mask=False, *,
                                                  scale=None):
    """reference :4211-4248: output laid out like the query, the real float32 log-sum-exp (the
    backward op needs it) and the placeholders of ATen's 9-value contract."""
    ops = None if return_debug_mask else _flash_operands(query, key, value, dropout_p, scale)
    if ops is None:
        return NOT_HANDLED
    q, k, v, s = ops
    out, lse = hip_ops.attention(q._holder, k._holder, v._holder, s, bool(is_causal),
                                 return_lse=True, like_query=True)
    seed = torch.zeros((), dtype=torch.int64, device=out.device)
    return (_wrap(out), _wrap(lse), None, None, q._shape[2], k._shape[2], _wrap(seed),
            _wrap(seed.clone()), _wrap(torch.empty(0, dtype=out.dtype, device=out.device)))


def fast_aten__scaled_dot_product_flash_attention_backward(grad_out, query, key, value, out,
                                                           logsumexp, cum_seq_q, cum_seq_k, max_q,
                                                           max_k, dropout_p, is_causal,
                                                           philox_seed, philox_offset, *,
                                                           scale=None):
    """reference :4251-4338 and :4089-4170: (grad_query, grad_key, grad_value) from the fused
    backward kernels; a log-sum-exp view that is not contiguous is materialised first."""
    ops = _flash_operands(query, key, value, dropout_p, scale)
    g, o, lse = _t(grad_out), _t(out), _t(logsumexp)
    if ops is None or g is None or o is None or lse is None or cum_seq_q is not None \
            or cum_seq_k is not None:
        return NOT_HANDLED
    q, k, v, s = ops
    lse_h = lse._holder if lse._holder.is_contiguous() else lse._holder.contiguous()
    if not hip_ops.attention_backward_supported(g._holder, q._holder, k._holder, v._holder,
                                                o._holder, lse_h):
        return NOT_HANDLED
    grads = hip_ops.attention_backward(g._holder, q._holder, k._holder, v._holder, o._holder,
                                       lse_h, s, bool(is_causal), packed=True)
    return tuple(_wrap(x) for x in grads)


# ---------------------------------------------------------------------------
# Layer norm (reference :2704-2794)
# ---------------------------------------------------------------------------
def fast_aten_native_layer_norm(input, normalized_shape, weight, bias, eps):
    a = _t(input)
    normalized_shape = tuple(int(s) for s in normalized_shape)
    k = len(normalized_shape)
    if a is None or a._numel == 0 or a._dtype not in _FLOAT_DTYPES or k < 1 \
            or len(a._shape) < k or tuple(a._shape[-k:]) != normalized_shape:
        return NOT_HANDLED
    gamma = beta = None
    if weight is not None:
        gamma = _t(weight)
        if gamma is None or gamma._dtype != a._dtype or gamma._device != a._device \
                or tuple(gamma._shape) != normalized_shape:
            return NOT_HANDLED
    if bias is not None:
        beta = _t(bias)
        if beta is None or beta._dtype != a._dtype or beta._device != a._device \
                or tuple(beta._shape) != normalized_shape:
            return NOT_HANDLED
    out, mean, rstd = hip_ops.layer_norm(a._holder, normalized_shape,
                                         None if gamma is None else gamma._holder,
                                         None if beta is None else beta._holder, float(eps))
    return _wrap(out), _wrap(mean), _wrap(rstd)


def fast_aten_layer_norm(input, normalized_shape, weight=None, bias=None, eps=1e-5,
                         cudnn_enable=True):
    """aten::layer_norm registered whole: without a gradient nobody reads the row statistics, so
    neither buffer is allocated or written (the composite would call native_layer_norm and drop
    two of its three results)."""
    a = _t(input)
    gamma = None if weight is None else _t(weight)
    beta = None if bias is None else _t(bias)
    if a is None or (weight is not None and gamma is None) or (bias is not None and beta is None):
        return NOT_HANDLED
    try:
        out, _, _ = hip_ops.layer_norm(a._holder, tuple(normalized_shape),
                                       None if gamma is None else gamma._holder,
                                       None if beta is None else beta._holder, float(eps),
                                       need_stats=False)
    except (ValueError, TypeError):
        return NOT_HANDLED
    return _wrap(out)


# ---------------------------------------------------------------------------
# Reductions (reference :2944-3133)
# ---------------------------------------------------------------------------
def _norm_reduce_dims(dim, rank, empty_is_all):
    """Sorted unique normalised reduce dims, or None if invalid (reference :2944-2973)."""
    if dim is None:
        return list(range(rank))
    if isinstance(dim, int) and not isinstance(dim, bool):
        dims = [dim]
    elif isinstance(dim, (list, tuple)):
        dims = list(dim)
    else:
        return None
    if len(dims) == 0:
        return list(range(rank)) if empty_is_all else []
    seen, out = set(), []
    for d in dims:
        if not isinstance(d, int) or isinstance(d, bool) or not -rank <= d < rank:
            return None
        d %= rank
        if d in seen:
            return None
        seen.add(d)
        out.append(d)
    return sorted(out)


def _reduced_shape(shape, reduce_dims, keepdim):
    rset = set(reduce_dims)
    if keepdim:
        return tuple(1 if i in rset else s for i, s in enumerate(shape))
    return tuple(s for i, s in enumerate(shape) if i not in rset)


def _cast(t: TorchMojoTensor, dtype):
    if t._dtype == dtype:
        return t
    if t._dtype not in _CAST_DTYPES or dtype not in _CAST_DTYPES:
        return None
    return _wrap(t._holder.to(dtype))


def _reduce(a: TorchMojoTensor, rdims, keepdim, op):
    if a._numel == 0:
        return None
    if len(a._shape) == 0:
        return _wrap(hip_ops.reduce(a._holder.reshape(1), [0], False, op).reshape(()))
    return _wrap(hip_ops.reduce(a._holder, rdims, bool(keepdim), op))


def fast_aten_sum(input, dim=None, keepdim=False, *, dtype=None):
    a = _t(input)
    if a is None:
        return NOT_HANDLED
    if dtype is not None:
        a = _cast(a, dtype)
        if a is None:
            return NOT_HANDLED
    elif not a._dtype.is_floating_point and a._dtype != torch.int64:
        a = _cast(a, torch.int64)  # torch promotes bool/integer sums to int64
        if a is None:
            return NOT_HANDLED
    if a._dtype not in _FLOAT_DTYPES + (torch.int64,):
        return NOT_HANDLED
    rdims = _norm_reduce_dims(dim, len(a._shape), empty_is_all=True)
    if rdims is None:
        return NOT_HANDLED
    if a._numel == 0:  # empty reduction: torch defines it as 0 (reference :3033-3037)
        return fast_filled(_reduced_shape(a._shape, rdims, keepdim), 0, a._dtype, a._device)
    out = _reduce(a, rdims, keepdim, _ek.SUM)
    return out if out is not None else NOT_HANDLED


def fast_aten_mean(input, dim=None, keepdim=False, *, dtype=None):
    a = _t(input)
    if a is None:
        return NOT_HANDLED
    if dtype is not None:
        if dtype not in _FLOAT_DTYPES:
            return NOT_HANDLED
        a = _cast(a, dtype)
        if a is None:
            return NOT_HANDLED
    if a._dtype not in _FLOAT_DTYPES:
        return NOT_HANDLED
    rdims = _norm_reduce_dims(dim, len(a._shape), empty_is_all=True)
    if rdims is None:
        return NOT_HANDLED
    out = _reduce(a, rdims, keepdim, _ek.MEAN)
    return out if out is not None else NOT_HANDLED


def fast_aten_amax(input, dim=(), keepdim=False):
    a = _t(input)
    if a is None or a._dtype not in _ROW_REDUCE_DTYPES:
        return NOT_HANDLED
    rdims = _norm_reduce_dims(dim, len(a._shape), empty_is_all=True)
    if rdims is None:
        return NOT_HANDLED
    out = _reduce(a, rdims, keepdim, _ek.AMAX)
    return out if out is not None else NOT_HANDLED


def fast_aten_argmax(input, dim=None, keepdim=False):
    a = _t(input)
    if a is None or a._numel == 0 or a._dtype not in _ROW_REDUCE_DTYPES:
        return NOT_HANDLED
    rank = len(a._shape)
    if dim is None:
        return _wrap(hip_ops.argmax(a._holder, None, bool(keepdim)))
    if not (isinstance(dim, int) and not isinstance(dim, bool) and rank > 0 and -rank <= dim < rank):
        return NOT_HANDLED
    return _wrap(hip_ops.argmax(a._holder, dim % rank, bool(keepdim)))


def fast_aten_gelu(input, approximate="none"):
    a = _t(input)
    if a is None or a._dtype not in _FLOAT_DTYPES or approximate not in ("none", "tanh"):
        return NOT_HANDLED
    return _wrap(hip_ops.gelu(a._holder, approximate))


def fast_aten_embedding(input, weight, padding_idx=-1, scale_grad_by_freq=False, sparse=False):
    """``input`` is the table and ``weight`` the indices (aten naming, reference :5336-5371)."""
    table, idx = _t(input), _t(weight)
    if table is None or idx is None or table._device != idx._device \
            or table._dtype not in _FLOAT_DTYPES or idx._dtype not in (torch.int32, torch.int64) \
            or len(table._shape) != 2 or (table._shape[0] == 0 and idx._numel > 0):
        return NOT_HANDLED
    return _wrap(hip_ops.embedding(table._holder, idx._holder))


# ---------------------------------------------------------------------------
# Backward twins (reference :1413-1447, :2797-2913, :3237-3330, :4939-5031)
# ---------------------------------------------------------------------------
def fast_aten_gelu_backward(grad_output, self, *, approximate="none"):
    grad, a = _t(grad_output), _t(self)
    if approximate not in ("none", "tanh") or grad is None or a is None \
            or not _same_device(grad, a) or grad._dtype != a._dtype \
            or a._dtype not in _FLOAT_DTYPES or tuple(grad._shape) != tuple(a._shape):
        return NOT_HANDLED
    return _wrap(hip_ops.gelu_backward(grad._holder, a._holder, approximate))


def _softmax_backward_data(grad_output, output, dim, input_dtype, log):
    grad, saved = _t(grad_output), _t(output)
    if grad is None or saved is None or tuple(grad._shape) != tuple(saved._shape) \
            or grad._dtype != saved._dtype or not _same_device(grad, saved) \
            or grad._dtype not in _FLOAT_DTYPES or input_dtype not in _FLOAT_DTYPES \
            or not isinstance(dim, int) or isinstance(dim, bool):
        return NOT_HANDLED
    if grad._dtype != input_dtype and not (grad._dtype == torch.float32
                                           and input_dtype == torch.float16):
        return NOT_HANDLED
    rank = len(grad._shape)
    if rank == 0:
        if dim not in (-1, 0):
            return NOT_HANDLED
    elif not -rank <= dim < rank:
        return NOT_HANDLED
    result = hip_ops.softmax_backward(grad._holder, saved._holder, dim, log)
    return _wrap(result if result.dtype == input_dtype else result.to(input_dtype))


def fast_aten__log_softmax_backward_data(grad_output, output, dim, input_dtype):
    return _softmax_backward_data(grad_output, output, dim, input_dtype, True)


def fast_aten__softmax_backward_data(grad_output, output, dim, input_dtype):
    return _softmax_backward_data(grad_output, output, dim, input_dtype, False)


def fast_aten_native_layer_norm_backward(grad_out, input, normalized_shape, mean, rstd, weight,
                                         bias, output_mask):
    """Everything is validated from metadata before anything is materialised or allocated
    (reference :2797-2813)."""
    grad, a, saved_mean, saved_rstd = _t(grad_out), _t(input), _t(mean), _t(rstd)
    gamma = _t(weight) if weight is not None else None
    beta = _t(bias) if bias is not None else None
    normalized_shape = tuple(int(s) for s in normalized_shape)
    mask = tuple(output_mask)
    k = len(normalized_shape)
    if len(mask) != 3 or any(not isinstance(m, bool) for m in mask) or grad is None or a is None \
            or saved_mean is None or saved_rstd is None or a._dtype not in _FLOAT_DTYPES \
            or grad._dtype != a._dtype or saved_mean._dtype != torch.float32 \
            or saved_rstd._dtype != torch.float32 \
            or not _same_device(grad, a, saved_mean, saved_rstd, gamma, beta) \
            or tuple(grad._shape) != tuple(a._shape) or k < 1 or len(a._shape) < k \
            or tuple(a._shape[-k:]) != normalized_shape:
        return NOT_HANDLED
    cols = math.prod(normalized_shape)
    if cols <= 0:
        return NOT_HANDLED
    rows = a._numel // cols
    if saved_mean._numel != rows or saved_rstd._numel != rows:
        return NOT_HANDLED
    for given, t in ((weight, gamma), (bias, beta)):
        if given is not None and (t is None or t._dtype != a._dtype
                                  or tuple(t._shape) != normalized_shape):
            return NOT_HANDLED
    if (mask[1] and gamma is None) or (mask[2] and beta is None):
        return NOT_HANDLED
    if not any(mask):
        return None, None, None
    dx, dw, db = hip_ops.layer_norm_backward(
        grad._holder, a._holder, normalized_shape, saved_mean._holder, saved_rstd._holder,
        None if gamma is None else gamma._holder, mask)
    return tuple(None if t is None else _wrap(t) for t in (dx, dw, db))


def fast_aten_linear_backward(self, grad_output, weight, output_mask):
    a, grad, w = _t(self), _t(grad_output), _t(weight)
    mask = tuple(output_mask)
    if len(mask) != 3 or any(not isinstance(m, bool) for m in mask) or a is None or grad is None \
            or w is None or not _same_device(a, grad, w) or a._dtype not in _FLOAT_DTYPES \
            or grad._dtype != a._dtype or w._dtype != a._dtype or len(w._shape) != 2 \
            or len(a._shape) < 1 or a._shape[-1] != w._shape[1] or grad._shape[-1] != w._shape[0] \
            or tuple(grad._shape[:-1]) != tuple(a._shape[:-1]):
        return NOT_HANDLED
    dx, dw, db = hip_ops.linear_backward(a._holder, grad._holder, w._holder, mask)
    return tuple(None if t is None else _wrap(t) for t in (dx, dw, db))


# ---------------------------------------------------------------------------
# Call counting under TORCH_MOJO_BACKEND_TESTING=1 (reference :5499-5522)
# ---------------------------------------------------------------------------
def _instrument_call_counts():
    module = globals()
    for name, fn in list(module.items()):
        if not (name.startswith("fast_aten") or name.startswith("_fast_aten")) or not callable(fn):
            continue

        def make(fn):
            @functools.wraps(fn)
            def counted(*args, **kwargs):
                counted.call_count += 1
                return fn(*args, **kwargs)

            counted.call_count = 0
            return counted

        module[name] = make(fn)


if torch_mojo_backend.is_running_tests.IS_RUNNING_TESTS:
    _instrument_call_counts()
