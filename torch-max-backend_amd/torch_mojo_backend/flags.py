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


def hip_graph() -> bool:
    """Inference graphs over HIP tensors: after one ordinary run per set of input shapes the step
    program is captured into a HIP graph and later calls replay it (one graph launch instead of a
    Python step per node; a launch-bound forward such as GPT-2 small at batch 1 runs several times
    faster). Inputs whose address changes from call to call are copied into buffers the graph
    owns, results are handed out as copies. Off by default: the graph keeps the memory of one
    whole run, and what the steps decide on the host while it is recorded (a mask buffer found to
    be causal) stays decided until an input's address, shape or version counter changes. The
    reference has no counterpart (MAX compiles the whole graph; its executor is one call,
    torch_compile_backend/compiler.py:455-532)."""
    return _flag("HIP_GRAPH")
