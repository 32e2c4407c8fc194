"""Autograd over eager ``mojo`` tensors.

``TorchMojoTensor`` is a wrapper subclass, so PyTorch's generated autograd applies whenever an op
has a derivative formula: the formulas run on mojo tensors and reach the backward twins of the hot
ops (``linear_backward``, ``native_layer_norm_backward``, ``gelu_backward``,
``_log_softmax_backward_data``, ``_softmax_backward_data``) through their PrivateUse1
registrations. What is left for this module are the ops PyTorch would normally *decompose* before
autograd sees them and which the eager device registers whole for speed (``softmax.int``,
``contiguous``, ``layer_norm``, ``scaled_dot_product_attention``): registered at the backend key they have no
derivative, so each gets an ``AutogradPrivateUse1`` kernel that takes the differentiable route
when a gradient is wanted and the registered fast kernel otherwise (the reference keeps the same
split in mojo_device/mojo_device_autograd.py:1-60).
"""

from __future__ import annotations

import math

import torch

from .torch_mojo_tensor import DIRECT_IMPLS, TorchMojoTensor

_registered = False
aten = torch.ops.aten


# the overloads the eager registry (and with it DIRECT_IMPLS) is keyed by
_SOFTMAX_INT = aten.softmax.int
_LOG_SOFTMAX_INT = aten.log_softmax.int
_CONTIGUOUS = aten.contiguous.default
_LAYER_NORM = aten.layer_norm.default
_SDPA = aten.scaled_dot_product_attention.default


def _wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(
        isinstance(t, torch.Tensor) and t.requires_grad for t in tensors)


_dispatch_modes_active = torch._C._len_torch_dispatch_stack


def _below_autograd(op, *args, **kwargs):
    """The registered kernel of `op` when no gradient is wanted. With real HIP holders behind the
    first argument the eager implementation is called directly (one Python entry per op, as
    without an autograd kernel); while torch.compile traces (stand-in holders) or for other
    argument types the call is redispatched below the autograd keys."""
    first = args[0]
    if type(first) is TorchMojoTensor and type(first._holder) is torch.Tensor \
            and _dispatch_modes_active() == 0:  # a mode (profiler, fake tensors) must see the op
        impl = DIRECT_IMPLS.get(op)
        if impl is not None:
            return impl(*args, **kwargs)
    with torch._C._AutoDispatchBelowAutograd():
        return op(*args, **kwargs)


def _softmax_int(self, dim, dtype=None):
    if _wants_grad(self):
        x = self if dtype is None or dtype == self.dtype else self.to(dtype)
        return aten._softmax(x, dim, False)          # has a derivative: _softmax_backward_data
    return _below_autograd(_SOFTMAX_INT, self, dim, dtype)


def _log_softmax_int(self, dim, dtype=None):
    if _wants_grad(self):
        x = self if dtype is None or dtype == self.dtype else self.to(dtype)
        return aten._log_softmax(x, dim, False)
    return _below_autograd(_LOG_SOFTMAX_INT, self, dim, dtype)


def _contiguous(self, *, memory_format=torch.contiguous_format):
    if _wants_grad(self):
        if self.is_contiguous(memory_format=memory_format):
            return aten.alias(self)
        return aten.clone(self, memory_format=memory_format)
    return _below_autograd(_CONTIGUOUS, self, memory_format=memory_format)


def _layer_norm(input, normalized_shape, weight=None, bias=None, eps=1e-5, cudnn_enable=True):
    if _wants_grad(input, weight, bias):
        return aten.native_layer_norm(input, normalized_shape, weight, bias, eps)[0]
    return _below_autograd(_LAYER_NORM, input, normalized_shape, weight, bias, eps, cudnn_enable)


def _fused_attention_takes(query, key, value, scale) -> bool:
    from torch_mojo_backend.eager_kernels import hip_ops

    if not all(isinstance(x, TorchMojoTensor) for x in (query, key, value)) or not scale > 0.0:
        return False
    return query.dim() == 4 and hip_ops.attention_supported(query._holder, key._holder, value._holder)


def _sdpa(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, *, scale=None,
          enable_gqa=False):
    if not _wants_grad(query, key, value):
        return _below_autograd(_SDPA, query, key, value, attn_mask, dropout_p, is_causal,
                               scale=scale, enable_gqa=enable_gqa)
    if dropout_p != 0.0 or enable_gqa:
        raise NotImplementedError("scaled_dot_product_attention with dropout or grouped-query "
                                  "attention has no gradient on the mojo device")
    s = float(scale) if scale is not None else 1.0 / math.sqrt(query.shape[-1])
    if attn_mask is None and _fused_attention_takes(query, key, value, s):
        # one fused forward that also returns the log-sum-exp; PyTorch's derivative formula of
        # this op calls _scaled_dot_product_flash_attention_backward, the fused backward
        return aten._scaled_dot_product_flash_attention(query, key, value, 0.0, bool(is_causal),
                                                        False, scale=s)[0]
    # the differentiable route: matmul, scale, mask, softmax, matmul (each with a derivative)
    scores = torch.matmul(query, key.transpose(-2, -1)) * s
    t, n = query.shape[-2], key.shape[-2]
    if is_causal:
        keep = torch.ones(t, n, dtype=torch.bool, device=query.device).tril()
        scores = scores.masked_fill(~keep, float("-inf"))
    if attn_mask is not None:
        if attn_mask.dtype == torch.bool:
            scores = scores.masked_fill(~attn_mask, float("-inf"))
        else:
            scores = scores + attn_mask
    return torch.matmul(aten._softmax(scores, -1, False), value)


_AUTOGRAD_KERNELS = {
    "aten::softmax.int": _softmax_int,
    "aten::log_softmax.int": _log_softmax_int,
    "aten::contiguous": _contiguous,
    "aten::layer_norm": _layer_norm,
    "aten::scaled_dot_product_attention": _sdpa,
}


def register_autograd_kernels(registered_ops) -> None:
    """AutogradPrivateUse1 kernels for those of the composite ops above that the device
    registers at its backend key (``registered_ops``: the names in the eager registry)."""
    global _registered
    if _registered:
        return
    for name, fn in _AUTOGRAD_KERNELS.items():
        if name in registered_ops:
            torch.library.impl(name, "AutogradPrivateUse1")(fn)
    _registered = True
