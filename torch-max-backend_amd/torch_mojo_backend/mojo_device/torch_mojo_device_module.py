"""The ``torch.mojo`` device module PyTorch expects from a PrivateUse1 backend
(reference: torch_mojo_backend/mojo_device/torch_mojo_device_module.py). ``mojo:i`` is HIP
device ``i``; synchronisation is the HIP device's. The module-level ``current_device`` is a
plain global, as in the reference (:7, :111-119)."""

from __future__ import annotations

import torch

_current_device = 0


def is_initialized() -> bool:
    return True


def is_available() -> bool:
    return torch.cuda.is_available()


def device_count() -> int:
    return torch.cuda.device_count()


def current_device() -> int:
    return _current_device


def set_device(device) -> None:
    global _current_device
    index = device if isinstance(device, int) else torch.device(device).index
    _current_device = int(index or 0)


def _is_in_bad_fork() -> bool:
    return False


def manual_seed_all(seed: int) -> None:
    torch.cuda.manual_seed_all(seed)


def synchronize(device=None) -> None:
    index = _current_device if device is None else (
        device if isinstance(device, int) else (torch.device(device).index or 0))
    torch.cuda.synchronize(index)


def get_amp_supported_dtype():
    return [torch.float16, torch.bfloat16]
