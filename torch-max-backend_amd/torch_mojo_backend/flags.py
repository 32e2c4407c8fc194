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
