"""``TorchMojoTensor``: the eager ``mojo`` tensor.

Same shape as the reference's class (torch_mojo_backend/mojo_device/torch_mojo_tensor.py:255-588):
a storage-less ``PrivateUse1`` wrapper subclass whose payload is a ``_holder`` owning the device
allocation plus layout metadata (``_ptr``, ``_shape``, ``_strides``, ``_offset``, ``_dtype``,
``_numel``, ``_itemsize``, ``_device``, ``_is_contiguous``; read-only properties here). Views share
the holder's allocation. Here the holder is a PyTorch-ROCm tensor (its caching allocator is
stream-ordered, the job the reference's ``TensorHolder`` does, op_utils/__init__.mojo:250-263),
already viewed with this tensor's shape/strides/offset, so kernels take ``_ptr`` directly.
"""

from __future__ import annotations

import torch

MAX_RANK = 8  # reference :243


# OpOverload -> the function registered for it on the mojo device. Filled by
# register_mojo_devices(); lets __torch_dispatch__ call the implementation directly instead of
# going through the dispatcher a second time (about a third of the per-op host cost).
DIRECT_IMPLS: dict = {}

_MOJO_DEVICES: dict = {}
_MOJO_OF_HIP: dict = {}  # HIP device of a holder -> the mojo device of its wrapper


def _mojo_device(index: int) -> torch.device:
    dev = _MOJO_DEVICES.get(index)
    if dev is None:
        dev = _MOJO_DEVICES[index] = torch.device("mojo", index)
    return dev


_make_wrapper = torch.Tensor._make_wrapper_subclass
_STRIDED = torch.strided


class TorchMojoTensor(torch.Tensor):
    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        # Let higher-priority wrappers (FakeTensor, FunctionalTensor) handle mixed calls, then
        # continue into the mojo implementation of the exact overload PyTorch chose.
        if len(types) != 1 or types[0] is not cls:
            for t in types:
                if t is not cls and not issubclass(cls, t):
                    return NotImplemented
        # torch.compile traces through this class with stand-in (fake / functional) holders: no
        # kernel can take those, the op is replayed on the holders instead (see _trace_dispatch)
        for a in args:
            if type(a) is cls:
                if type(a._holder) is not torch.Tensor:
                    return cls._trace_dispatch(func, args, kwargs or {})
                break
        impl = DIRECT_IMPLS.get(func)
        if impl is not None:
            # the implementations work on the HIP holders, so nothing below re-enters this method
            return impl(*args, **kwargs) if kwargs else impl(*args)
        with torch._C._DisableTorchDispatch():
            return func(*args, **(kwargs or {}))

    @classmethod
    def _wrap(cls, holder: torch.Tensor) -> "TorchMojoTensor":
        """Adopt a HIP tensor (zero-copy) as a mojo tensor with the same view."""
        device = holder.device
        if device.type != "cuda":
            raise TypeError(f"a mojo tensor is backed by HIP memory, got {device}")
        shape = holder.shape
        if len(shape) > MAX_RANK:
            raise NotImplementedError(f"mojo tensors support at most rank {MAX_RANK}, got {len(shape)}")
        if holder.requires_grad or holder.grad_fn is not None:
            holder = holder.detach()
        # positional (size, strides, storage_offset, memory_format, dtype, layout, device,
        # pin_memory): keyword parsing is a quarter of this call, which runs once per eager op
        res = _make_wrapper(cls, shape, holder.stride(), holder.storage_offset(), None, holder.dtype,
                            _STRIDED, _mojo_device(device.index or 0), False)
        # This runs once per eager op: only the holder is stored, the layout attributes below
        # are read from it when an implementation asks for them.
        res._holder = holder
        return res

    @classmethod
    def _adopt(cls, holder: torch.Tensor) -> "TorchMojoTensor":
        """`_wrap` for what an implementation on this device has just computed from holders: a
        HIP tensor outside any autograd graph by construction, so only the rank is checked."""
        shape = holder.shape
        if len(shape) > MAX_RANK:
            raise NotImplementedError(f"mojo tensors support at most rank {MAX_RANK}, got {len(shape)}")
        hip = holder.device
        dev = _MOJO_OF_HIP.get(hip)
        if dev is None:
            dev = _MOJO_OF_HIP[hip] = _mojo_device(hip.index or 0)
        res = _make_wrapper(cls, shape, holder.stride(), holder.storage_offset(), None, holder.dtype,
                            _STRIDED, dev, False)
        res._holder = holder
        return res

    # torch.compile support: as a traceable wrapper subclass the tensor flattens to its HIP holder,
    # so a compiled graph computes on the holders (zero-copy) and AOTAutograd wraps its outputs
    # back into mojo tensors.
    def __tensor_flatten__(self):
        return ["_holder"], None

    @staticmethod
    def __tensor_unflatten__(inner_tensors, meta, outer_size, outer_stride):
        return TorchMojoTensor._wrap(inner_tensors["_holder"])

    @classmethod
    def _trace_dispatch(cls, func, args, kwargs):
        """The op on the holders, results wrapped again: what tracing records for an op on mojo
        tensors (device arguments naming the mojo device become the holders' HIP device)."""
        from torch.utils._pytree import tree_map

        hip = [None]

        def unwrap(x):
            if isinstance(x, cls):
                hip[0] = x._holder.device
                return x._holder
            return x

        a, kw = tree_map(unwrap, args), tree_map(unwrap, kwargs)
        if isinstance(kw.get("device"), torch.device) and kw["device"].type == "mojo":
            kw["device"] = hip[0] or hip_device_of(kw["device"])
        out = func(*a, **kw)
        return tree_map(lambda t: cls._wrap(t) if isinstance(t, torch.Tensor) and t.device.type == "cuda"
                        else t, out)

    def __coerce_same_metadata_as_tangent__(self, expected_meta, expected_type=None):
        return self if expected_type in (None, torch.Tensor, TorchMojoTensor) else None

    # Layout metadata of the reference's class (:255-337), derived from the holder.
    _ptr = property(lambda self: self._holder.data_ptr())
    _shape = property(lambda self: tuple(self._holder.shape))
    _strides = property(lambda self: tuple(self._holder.stride()))
    _offset = property(lambda self: self._holder.storage_offset())
    _dtype = property(lambda self: self._holder.dtype)
    _itemsize = property(lambda self: self._holder.element_size())
    _numel = property(lambda self: self._holder.numel())
    _device = property(lambda self: self._holder.device)
    _is_contiguous = property(lambda self: self._holder.is_contiguous())

    @classmethod
    def _alloc(cls, shape, dtype: torch.dtype, device) -> "TorchMojoTensor":
        """A new contiguous uninitialised tensor (one device allocation)."""
        return cls._wrap(torch.empty(tuple(shape), dtype=dtype, device=hip_device_of(device)))

    def __reduce_ex__(self, protocol):
        # Pickles as a plain CPU tensor (reference :498-509).
        return self._holder.cpu().__reduce_ex__(protocol)

    def __repr__(self, *, tensor_contents=None):
        return f"TorchMojoTensor({self._holder.cpu()!r}, device='{self.device}')"


def hip_device_of(device) -> torch.device:
    """``mojo:i`` (or an int, or a HIP device) -> the HIP device backing it."""
    if isinstance(device, int):
        return torch.device("cuda", device)
    device = torch.device(device)
    if device.type == "cuda":
        return device
    if device.type == "mojo":
        index = device.index or 0
        if index >= max(torch.cuda.device_count(), 1):
            raise RuntimeError(
                f"{device} does not name a HIP device; the CPU entry of get_accelerators() has "
                "no kernels in this build")
        return torch.device("cuda", index)
    raise TypeError(f"not a mojo device: {device}")
