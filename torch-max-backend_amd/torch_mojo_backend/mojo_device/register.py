"""``register_mojo_devices()``: enable the eager ``mojo`` device
(reference: torch_mojo_backend/mojo_device/register.py:141-198)."""

from __future__ import annotations

import torch

_registered = False


def register_mojo_devices() -> None:
    """Rename PrivateUse1 to ``mojo``, install the device module and register every collected
    aten op with ``torch.library.impl(op_name, "privateuseone")`` (reference :180-181)."""
    global _registered
    if _registered:
        return
    from torch.utils.backend_registration import _setup_privateuseone_for_python_backend

    from . import torch_mojo_device_module
    from .mojo_device_aten_ops import _aten_ops_registry

    # Tied parameters (GPT-2's wte / lm_head) must stay one Parameter through .to("mojo").
    torch.__future__.set_swap_module_params_on_conversion(True)
    _setup_privateuseone_for_python_backend("mojo", backend_module=torch_mojo_device_module)
    from .mojo_device_aten_ops import _resolve_overload
    from .torch_mojo_tensor import DIRECT_IMPLS

    for op_name, func in _aten_ops_registry:
        torch.library.impl(op_name, "privateuseone")(func)
        # "aten::mean" names the default overload, as torch.library resolves it
        DIRECT_IMPLS[_resolve_overload(op_name)] = func
    from .mojo_device_autograd import register_autograd_kernels

    register_autograd_kernels({name for name, _ in _aten_ops_registry})
    _registered = True
