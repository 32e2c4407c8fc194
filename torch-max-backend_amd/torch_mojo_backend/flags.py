"""Environment switches of the backend (same variable names as the reference,
torch_mojo_backend/flags.py:6-33, including the ``PYTORCH_`` aliases)."""

import os

POSITIVE_VALUES = ("1", "true", "yes")


def _flag(name: str) -> bool:
    for prefix in ("TORCH_MOJO_BACKEND_", "PYTORCH_MOJO_BACKEND_"):
        if os.environ.get(prefix + name, "0").lower() in POSITIVE_VALUES:
            return True
    return False


def profiling_enabled() -> bool:
    """Print graph build / run wall times."""
    return _flag("PROFILE")


def verbose_enabled() -> bool:
    """Print the FX graph and the op histogram at compile time."""
    return _flag("VERBOSE")


def debug_graph() -> bool:
    """Compare every node's output with the same aten op run by PyTorch-ROCm itself."""
    return _flag("DEBUG_GRAPH")


def round_like_unfused() -> bool:
    """Fused steps (GEMM + GELU, GEMM + residual add) round to the storage type wherever the
    separate kernels would have stored a tensor, which makes a fused graph bit-identical to the
    unfused one. Off by default: a fused epilogue stays in float32 up to its one cast, and a
    16-bit graph keeps its residual stream in float32 between the blocks."""
    return _flag("ROUND_LIKE_UNFUSED")


def cache_host_parameters() -> bool:
    """Graphs over host tensors: keep the device copy of each ``nn.Parameter`` between calls
    (revalidated by data pointer and version counter). Off by default, because writes that
    bypass the version counter (``p.data.mul_()``, writes through ``p.numpy()``) would keep the
    stale copy in use; with the switch off every call uploads what the host tensors hold at that
    moment, as the reference's aliasing buffer import sees them
    (torch_compile_backend/compiler.py:535-566)."""
    return _flag("CACHE_HOST_PARAMETERS")
