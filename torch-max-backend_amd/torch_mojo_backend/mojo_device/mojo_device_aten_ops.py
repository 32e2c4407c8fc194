"""Eager ``mojo`` device op registrations.

Same mechanism as the reference's ``mojo_device/mojo_device_aten_ops.py``:
``register_aten_op(name)`` collects ``(op_name, fn)`` pairs (:42-64) that
``register_mojo_devices()`` hands to ``torch.library.impl(op_name, "privateuseone")``;
``_register_fast(op_name, fast_name)`` binds an op lazily to ``aten_fast.<fast_name>`` and
raises ``NotImplementedError`` naming the op when that returns ``NOT_HANDLED`` (:84-135).

Hot ops go to the HIP kernels through ``aten_fast``. The handful of runtime ops a tensor needs
to exist at all (allocation, host/device copies, zero-copy views) act on the holder directly.
"""

from __future__ import annotations

import functools
from collections.abc import Callable

import torch

import torch_mojo_backend.is_running_tests
from torch_mojo_backend.mojo_device.torch_mojo_tensor import TorchMojoTensor, hip_device_of

_aten_ops_registry: list = []
EAGER_CALL_COUNTERS: dict = {}


def register_aten_op(op_name: str):
    """Decorator marking a function as the ``mojo`` implementation of ``op_name``."""

    def decorator(func: Callable) -> Callable:
        if torch_mojo_backend.is_running_tests.IS_RUNNING_TESTS:

            @functools.wraps(func)
            def counted(*args, **kwargs):
                counted.call_count += 1
                return func(*args, **kwargs)

            counted.call_count = 0
            EAGER_CALL_COUNTERS[op_name] = counted
            _aten_ops_registry.append((op_name, counted))
            return counted
        _aten_ops_registry.append((op_name, func))
        return func

    return decorator


_aten_fast_module = None


def _fast():
    global _aten_fast_module
    if _aten_fast_module is None:
        from torch_mojo_backend.eager_kernels import aten_fast

        _aten_fast_module = aten_fast
    return _aten_fast_module


def _describe_args(args, kwargs) -> str:
    descs = []
    for a in list(args) + list(kwargs.values()):
        if isinstance(a, TorchMojoTensor):
            descs.append(f"{tuple(a._shape)}:{a._dtype}")
        elif isinstance(a, torch.Tensor):
            descs.append(f"{tuple(a.shape)}:{a.dtype}:{a.device}")
    return ", ".join(descs) or "none"


def _unsupported(op_name: str, args=(), kwargs=None) -> NotImplementedError:
    return NotImplementedError(
        f"{op_name} is not supported by mojo eager mode for these inputs "
        f"(tensor args: {_describe_args(args, kwargs or {})}). There is no fallback; add a fast "
        "kernel in torch_mojo_backend/eager_kernels/ or open an issue."
    )


def _eager_impl(fast_name: str, op_name: str) -> Callable:
    """Bind an op to its aten_fast implementation; raise on NOT_HANDLED."""
    fast_fn = None
    not_handled = None

    def dispatcher(*args, **kwargs):
        nonlocal fast_fn, not_handled
        if fast_fn is None:
            aten_fast = _fast()
            fast_fn = getattr(aten_fast, fast_name)
            not_handled = aten_fast.NOT_HANDLED
        result = fast_fn(*args, **kwargs)
        if result is not_handled:
            raise _unsupported(op_name, args, kwargs)
        return result

    return dispatcher


def _not_implemented(op_name: str) -> Callable:
    def raiser(*args, **kwargs):
        raise _unsupported(op_name, args, kwargs)

    return raiser


def _register_fast(op_name: str, fast_name: str):
    register_aten_op(op_name)(_eager_impl(fast_name, op_name))


def _register_missing(op_name: str):
    register_aten_op(op_name)(_not_implemented(op_name))


# ---------------------------------------------------------------------------
# The hot ops (same op names as the reference registers, :860-1021)
# ---------------------------------------------------------------------------
_register_fast("aten::_log_softmax", "fast_aten__log_softmax")
_register_fast("aten::_softmax", "fast_aten__softmax")
_register_fast("aten::addmm", "fast_aten_addmm")
_register_fast("aten::amax", "fast_aten_amax")
_register_fast("aten::argmax", "fast_aten_argmax")
_register_fast("aten::bmm", "fast_aten_bmm")
_register_fast("aten::gelu", "fast_aten_gelu")
_register_fast("aten::embedding", "fast_aten_embedding")
_register_fast("aten::linear", "fast_aten_linear")
_register_fast("aten::mean", "fast_aten_mean")
_register_fast("aten::mean.dim", "fast_aten_mean")
_register_fast("aten::mm", "fast_aten_mm")
_register_fast("aten::native_layer_norm", "fast_aten_native_layer_norm")
_register_fast("aten::layer_norm", "fast_aten_layer_norm")
_register_fast("aten::scaled_dot_product_attention", "fast_aten_scaled_dot_product_attention")
_register_fast("aten::_scaled_dot_product_flash_attention",
               "fast_aten__scaled_dot_product_flash_attention")
_register_fast("aten::_scaled_dot_product_flash_attention_backward",
               "fast_aten__scaled_dot_product_flash_attention_backward")  # reference :881-882
_register_fast("aten::softmax.int", "fast_aten_softmax")
_register_fast("aten::cat", "fast_aten_cat")  # reference :914
_register_fast("aten::sum.dim_IntList", "fast_aten_sum")
# backward twins (reference :930-1000 registers the same op names)
_register_fast("aten::gelu_backward", "fast_aten_gelu_backward")
_register_fast("aten::_log_softmax_backward_data", "fast_aten__log_softmax_backward_data")
_register_fast("aten::_softmax_backward_data", "fast_aten__softmax_backward_data")
_register_fast("aten::native_layer_norm_backward", "fast_aten_native_layer_norm_backward")
_register_fast("aten::linear_backward", "fast_aten_linear_backward")


def _out_variant(op_name: str, fast_name: str, *, dtype_policy: str = "safe_cast"):
    """An ``out=`` overload from the functional implementation: compute, check the destination,
    then a strided, casting copy into ``out`` (reference :155-207). ``dtype_policy``:
    "safe_cast" (``torch.can_cast(result, out)``), "exact", or "bool_or_uint8". A destination of
    another shape is an error here (the reference resizes its payload; a wrapper over a HIP
    tensor cannot change its sizes)."""
    if dtype_policy not in ("safe_cast", "exact", "bool_or_uint8"):
        raise AssertionError(f"unknown out dtype policy: {dtype_policy}")

    def dispatcher(*args, out, **kwargs):
        if not isinstance(out, TorchMojoTensor):
            raise RuntimeError(f"{op_name}: expected out to be a mojo tensor")
        input_device = next((a._device for a in args if isinstance(a, TorchMojoTensor)), None)
        if input_device is not None and out._device != input_device:
            raise RuntimeError(f"{op_name}: expected out and input tensors to be on the same device")
        aten_fast = _fast()
        result = getattr(aten_fast, fast_name)(*args, **kwargs)
        if result is aten_fast.NOT_HANDLED:
            raise _unsupported(op_name, args, kwargs)
        if out._device != result._device:
            raise RuntimeError(f"{op_name}: expected out and result tensors to be on the same device")
        if dtype_policy == "exact":
            valid = result._dtype == out._dtype
        elif dtype_policy == "bool_or_uint8":
            valid = out._dtype in (torch.bool, torch.uint8)
        else:
            valid = torch.can_cast(result._dtype, out._dtype)
        if not valid:
            raise RuntimeError(f"result type {result._dtype} can't be cast to the desired output "
                               f"type {out._dtype}")
        if tuple(result._shape) != tuple(out._shape):
            raise RuntimeError(f"{op_name}: out has shape {tuple(out._shape)}, the result has "
                               f"{tuple(result._shape)}; resizing a mojo tensor is not supported")
        out._holder.copy_(result._holder)   # casts and follows out's strides
        return out

    return dispatcher


# out= overloads of the hot ops (the reference registers aten::mean.out, :761; the others share
# its machinery)
for _op, _fast_name, _policy in (
        ("aten::mean.out", "fast_aten_mean", "safe_cast"),
        ("aten::sum.IntList_out", "fast_aten_sum", "safe_cast"),
        ("aten::amax.out", "fast_aten_amax", "exact"),
        ("aten::argmax.out", "fast_aten_argmax", "exact"),
        ("aten::mm.out", "fast_aten_mm", "exact"),
        ("aten::bmm.out", "fast_aten_bmm", "exact"),
        ("aten::addmm.out", "fast_aten_addmm", "exact"),
        ("aten::_softmax.out", "fast_aten__softmax", "exact"),
        ("aten::_log_softmax.out", "fast_aten__log_softmax", "exact"),
        ("aten::gelu.out", "fast_aten_gelu", "exact")):
    register_aten_op(_op)(_out_variant(_op, _fast_name, dtype_policy=_policy))


@register_aten_op("aten::sum")
def _sum_default(self, *, dtype=None):
    result = _fast().fast_aten_sum(self, None, False, dtype=dtype)
    if result is _fast().NOT_HANDLED:
        raise _unsupported("aten::sum", (self,), {})
    return result


# ---------------------------------------------------------------------------
# Runtime plumbing: allocation, copies, views (act on the holder; no arithmetic)
# ---------------------------------------------------------------------------
def _holder(x):
    return x._holder if isinstance(x, TorchMojoTensor) else x


@register_aten_op("aten::empty.memory_format")
def _empty(size, *, dtype=None, layout=None, device=None, pin_memory=None, memory_format=None):
    dtype = dtype or torch.get_default_dtype()
    return TorchMojoTensor._wrap(torch.empty(tuple(size), dtype=dtype, device=hip_device_of(device)))


@register_aten_op("aten::empty_strided")
def _empty_strided(size, stride, *, dtype=None, layout=None, device=None, pin_memory=None):
    dtype = dtype or torch.get_default_dtype()
    return TorchMojoTensor._wrap(
        torch.empty_strided(tuple(size), tuple(stride), dtype=dtype, device=hip_device_of(device)))


@register_aten_op("aten::_copy_from")
def _copy_from(self, dst, non_blocking=False):
    """copy_(dst, self): host -> mojo, mojo -> host, mojo -> mojo."""
    src_h, dst_h = _holder(self), _holder(dst)
    dst_h.copy_(src_h, non_blocking=bool(non_blocking))
    return dst


@register_aten_op("aten::_to_copy")
def _to_copy(self, *, dtype=None, layout=None, device=None, pin_memory=None, non_blocking=False,
             memory_format=None):
    src = _holder(self)
    target = torch.device(device) if device is not None else self.device
    dtype = dtype or src.dtype
    if target.type == "mojo":
        return TorchMojoTensor._wrap(src.to(device=hip_device_of(target), dtype=dtype, copy=True))
    return src.to(device=target, dtype=dtype, copy=True)


@register_aten_op("aten::_local_scalar_dense")
def _local_scalar_dense(self):
    return self._holder.item()


def _view_op(op_name: str, fn: Callable):
    adopt = TorchMojoTensor._adopt

    @register_aten_op(op_name)
    def view(self, *args, **kwargs):
        return adopt(fn(self._holder, *args, **kwargs))

    return view


def _direct_view_ops():
    """view and transpose are two thirds of the views of a decode step: no lambda in between."""
    adopt = TorchMojoTensor._adopt

    @register_aten_op("aten::view")
    def view(self, size):
        return adopt(self._holder.view(size))

    @register_aten_op("aten::_unsafe_view")
    def unsafe_view(self, size):
        return adopt(self._holder.view(size))

    @register_aten_op("aten::transpose.int")
    def transpose(self, dim0, dim1):
        return adopt(self._holder.transpose(dim0, dim1))


_direct_view_ops()
_view_op("aten::_reshape_alias", lambda h, size, stride: h.as_strided(size, stride))
_view_op("aten::as_strided", lambda h, size, stride, storage_offset=None:
         h.as_strided(size, stride, h.storage_offset() if storage_offset is None else storage_offset))
_view_op("aten::t", lambda h: h.t())
_view_op("aten::permute", lambda h, dims: h.permute(dims))
_view_op("aten::expand", lambda h, size, implicit=False: h.expand(size))
_view_op("aten::unsqueeze", lambda h, dim: h.unsqueeze(dim))
_view_op("aten::squeeze.dim", lambda h, dim: h.squeeze(dim))
_view_op("aten::select.int", lambda h, dim, index: h.select(dim, index))
_view_op("aten::slice.Tensor", lambda h, dim=0, start=None, end=None, step=1:
         h[(slice(None),) * (dim % max(h.dim(), 1)) + (slice(start, end, step),)])
_view_op("aten::alias", lambda h: h.alias() if hasattr(h, "alias") else h.view(h.shape))
_view_op("aten::detach", lambda h: h.detach())
_view_op("aten::clone", lambda h, memory_format=None:
         h.clone(memory_format=memory_format if memory_format is not None else torch.preserve_format))


# ---------------------------------------------------------------------------
# Cold ops: everything else a GPT-2 forward or a greedy `generate` loop touches (elementwise
# arithmetic, comparisons, indexing, concatenation, factories). The reference gives each of them
# a Mojo kernel of its own (e.g. `Gather0` aten_fast.py:5336-5371, `AddF32Bf16Spec` :657-687);
# here they run as the PyTorch-ROCm kernel of the same op on the holders, exactly as the graph
# surface registers its non-hot ops. An op that is not listed still raises NotImplementedError.
# ---------------------------------------------------------------------------
def _resolve_overload(op_name: str):
    qual, _, overload = op_name.partition(".")
    namespace, _, name = qual.partition("::")
    packet = getattr(getattr(torch.ops, namespace), name)
    return getattr(packet, overload or "default")


_PLAIN_ARG_TYPES = frozenset((int, float, bool, str, type(None), torch.dtype, torch.memory_format,
                              torch.layout))


def _unwrap_arg(x, owners: list):
    """Nested / uncommon arguments: lists of tensors, mojo devices."""
    if isinstance(x, TorchMojoTensor):
        owners.append(x)
        return x._holder
    if isinstance(x, (list, tuple)):
        return type(x)(_unwrap_arg(y, owners) for y in x)
    if isinstance(x, torch.device) and x.type == "mojo":
        return hip_device_of(x)
    return x


def _wrap_result(y, owners: list):
    if isinstance(y, torch.Tensor):
        for owner in owners:  # in-place and out= forms hand back one of the inputs
            if owner._holder is y:
                return owner
        return TorchMojoTensor._wrap(y)
    if isinstance(y, (list, tuple)):
        return type(y)(_wrap_result(z, owners) for z in y)
    return y


def holder_impl(op_name: str) -> Callable:
    """The op on the HIP holders of its mojo arguments; results are wrapped (an output that is
    one of the inputs' holders — in-place and out= forms — comes back as that input)."""
    op = None

    def impl(*args, **kwargs):
        nonlocal op
        if op is None:
            op = _resolve_overload(op_name)
        owners = []
        call = []
        for a in args:  # this loop runs once per cold eager op: plain cases first
            t = type(a)
            if t is TorchMojoTensor:
                owners.append(a)
                call.append(a._holder)
            elif t in _PLAIN_ARG_TYPES:
                call.append(a)
            else:
                call.append(_unwrap_arg(a, owners))
        if kwargs:
            out = op(*call, **{k: _unwrap_arg(v, owners) for k, v in kwargs.items()})
        else:
            out = op(*call)
        if type(out) is torch.Tensor:
            for owner in owners:
                if owner._holder is out:
                    return owner
            return TorchMojoTensor._wrap(out)
        return _wrap_result(out, owners)

    return impl


_HOLDER_OPS = (
    # elementwise arithmetic and activations
    "aten::add.Tensor", "aten::add.Scalar", "aten::add_.Tensor", "aten::sub.Tensor",
    "aten::sub.Scalar", "aten::rsub.Scalar", "aten::mul.Tensor", "aten::mul.Scalar",
    "aten::mul_.Tensor", "aten::div.Tensor", "aten::div.Scalar", "aten::neg", "aten::pow.Tensor_Scalar",
    "aten::tanh", "aten::exp", "aten::sqrt", "aten::rsqrt", "aten::sigmoid", "aten::relu",
    "aten::where.self", "aten::masked_fill.Scalar", "aten::masked_fill_.Scalar",
    "aten::masked_fill.Tensor", "aten::clamp", "aten::clamp_min",
    # comparisons and boolean logic
    "aten::eq.Scalar", "aten::eq.Tensor", "aten::ne.Scalar", "aten::ne.Tensor", "aten::lt.Scalar",
    "aten::lt.Tensor", "aten::le.Scalar", "aten::le.Tensor", "aten::gt.Scalar", "aten::gt.Tensor",
    "aten::ge.Scalar", "aten::ge.Tensor", "aten::bitwise_and.Tensor", "aten::bitwise_or.Tensor",
    "aten::bitwise_not", "aten::logical_not", "aten::any", "aten::any.dim", "aten::all",
    "aten::all.dim", "aten::isin.Tensor_Tensor", "aten::isin.Tensor_Scalar",
    # reductions that are not hot, scans, selection
    "aten::max", "aten::max.dim", "aten::min", "aten::cumsum", "aten::topk", "aten::sort",
    "aten::multinomial",
    # indexing, gathering, concatenation
    "aten::index_select", "aten::gather", "aten::index.Tensor",
    "aten::index_put_", "aten::stack",
    "aten::split_with_sizes", "aten::unbind.int", "aten::squeeze", "aten::flatten.using_ints",
    "aten::tril", "aten::triu", "aten::repeat", "aten::roll",
    # fills, copies and factories
    "aten::fill_.Scalar", "aten::fill_.Tensor", "aten::zero_", "aten::copy_", "aten::full",
    "aten::full_like", "aten::zeros", "aten::zeros_like", "aten::ones", "aten::ones_like",
    "aten::new_ones", "aten::new_zeros", "aten::new_full", "aten::new_empty",
    "aten::empty_like", "aten::arange", "aten::arange.start", "aten::arange.start_step",
    "aten::scalar_tensor", "aten::lift_fresh", "aten::contiguous",
    # what a training step adds: losses, their gradients, embedding and elementwise backward ops,
    # the optimizer's in-place arithmetic
    "aten::nll_loss_forward", "aten::nll_loss_backward", "aten::embedding_dense_backward",
    "aten::tanh_backward", "aten::sigmoid_backward", "aten::threshold_backward",
    "aten::mse_loss", "aten::mse_loss_backward", "aten::sub_.Tensor", "aten::div_.Tensor",
    "aten::mul_.Scalar", "aten::add_.Scalar", "aten::addcmul_", "aten::addcdiv_", "aten::sqrt_",
    "aten::lerp_.Scalar", "aten::log", "aten::sum_to_size",
)
# The elementwise ops a decode loop issues by the hundred per token (HF's tanh-GELU alone is
# eight of them per layer) skip the generic argument walk: tensor-with-tensor and
# tensor-with-number calls go to the torch function of the same op on the holders.
_LEAN_BINARY = {"aten::add.Tensor": torch.add, "aten::mul.Tensor": torch.mul,
                "aten::sub.Tensor": torch.sub, "aten::pow.Tensor_Scalar": torch.pow}
_LEAN_UNARY = {"aten::tanh": torch.tanh}


def _lean_binary(op_name: str, fn: Callable) -> Callable:
    generic = holder_impl(op_name)
    adopt = TorchMojoTensor._adopt

    def impl(self, other, *rest, **kwargs):
        if not rest and not kwargs and type(self) is TorchMojoTensor:
            t = type(other)
            if t is TorchMojoTensor:
                return adopt(fn(self._holder, other._holder))
            if t is float or t is int:
                return adopt(fn(self._holder, other))
        return generic(self, other, *rest, **kwargs)

    return impl


def _lean_unary(op_name: str, fn: Callable) -> Callable:
    generic = holder_impl(op_name)
    adopt = TorchMojoTensor._adopt

    def impl(self, *rest, **kwargs):
        if not rest and not kwargs and type(self) is TorchMojoTensor:
            return adopt(fn(self._holder))
        return generic(self, *rest, **kwargs)

    return impl


for _name in _HOLDER_OPS:
    if _name in _LEAN_BINARY:
        register_aten_op(_name)(_lean_binary(_name, _LEAN_BINARY[_name]))
    elif _name in _LEAN_UNARY:
        register_aten_op(_name)(_lean_unary(_name, _LEAN_UNARY[_name]))
    else:
        register_aten_op(_name)(holder_impl(_name))


@register_aten_op("aten::split.Tensor")
def _split_tensor(self, split_size, dim=0):
    adopt = TorchMojoTensor._adopt
    return [adopt(piece) for piece in self._holder.split(split_size, dim)]
