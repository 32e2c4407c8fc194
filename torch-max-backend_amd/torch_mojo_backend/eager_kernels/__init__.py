"""Loader of ``libtmb_hip.so``, the C-ABI library of hand-written gfx950 kernels.

Takes the place of the reference's lazy Mojo-extension loader
(torch_mojo_backend/eager_kernels/__init__.py:36-126): there the kernels are JIT-compiled
CPython extensions, here they are one prebuilt shared library bound with ctypes. Kernels are
enqueued on the caller's stream and never synchronise (reference: same file, lines 9-12).

There is no CPU or PyTorch fallback: if the library is missing, loading raises.
"""

from __future__ import annotations

import ctypes
import os

_CSRC = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "..", "csrc"))
# TORCH_MOJO_BACKEND_HIP_LIBRARY names another build of the library (a diagnostic variant made with
# `TMB_VARIANT=... sh build.sh ...`); unset, the library beside the sources is loaded.
LIBRARY_PATH = os.environ.get("TORCH_MOJO_BACKEND_HIP_LIBRARY") or os.path.join(_CSRC, "libtmb_hip.so")

F32, F16, BF16, I64, I32 = 0, 1, 2, 3, 4
SUM, MEAN, AMAX = 0, 1, 2
EPI_NONE, EPI_GELU_TANH, EPI_GELU_ERF = 0, 1, 2
EPI_ROUND_LIKE_UNFUSED = 0x100  # flag: fused steps round where separate kernels would store
ERR_INVALID_ARGUMENT, ERR_UNSUPPORTED, ERR_WORKSPACE, ERR_SCRATCH_LIMIT = -1, -2, -3, -4  # tmb_status (include/tmb_hip.h)

# Every symbol include/tmb_hip.h declares, with its ctypes signature.
_i64, _vp, _ci, _sz, _dbl = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_double
_flt = ctypes.c_float
SIGNATURES = {
    "tmb_version": (_ci, []),
    "tmb_status_string": (ctypes.c_char_p, [_ci]),
    "tmb_softmax_rows": (_ci, [_vp, _vp, _i64, _i64, _ci, _ci, _ci, _vp]),
    "tmb_softmax_rows_scaled": (_ci, [_vp, _vp, _i64, _i64, _ci, _flt, _ci, _i64, _vp]),
    "tmb_layer_norm_rows": (_ci, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _dbl, _ci, _ci, _vp]),
    "tmb_reduce_workspace_bytes": (_sz, [_i64, _i64, _ci]),
    "tmb_argmax_workspace_bytes": (_sz, [_i64, _i64, _ci]),
    "tmb_reduce_rows": (_ci, [_vp, _vp, _i64, _i64, _ci, _ci, _vp, _sz, _vp]),
    "tmb_reduce_rows_static": (_ci, [_vp, _vp, _i64, _i64, _ci, _ci, _vp]),
    "tmb_argmax_rows": (_ci, [_vp, _vp, _i64, _i64, _ci, _vp, _sz, _vp]),
    "tmb_gemm": (_ci, [_vp, _vp, _vp, _vp] + [_i64] * 10 + [_ci] * 4 + [_vp]),
    "tmb_gemm_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _ci]),
    "tmb_gemm_ws": (_ci, [_vp, _vp, _vp, _vp] + [_i64] * 10 + [_ci] * 4 + [_vp, _sz, _vp]),
    "tmb_gemm_residual": (_ci, [_vp, _vp, _vp, _vp, _vp] + [_i64] * 12 + [_ci] * 6 + [_vp]),
    "tmb_attention_fwd": (_ci, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _vp,
                                _vp, _flt, _ci, _ci, _ci, _vp]),
    "tmb_attention_bwd_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "tmb_attention_bwd": (_ci, [_vp] * 10 + [_i64] * 5 + [_vp] * 8 + [_flt, _ci, _ci, _vp]),
    "tmb_attention_decode": (_ci, [_vp] * 5 + [_i64] * 5 + [_vp] * 5 + [_flt, _ci, _ci, _vp]),
    "tmb_gelu": (_ci, [_vp, _vp, _i64, _ci, _ci, _vp]),
    "tmb_gather_rows": (_ci, [_vp, _vp, _vp, _i64, _i64, _i64, _ci, _ci, _vp]),
    "tmb_gelu_backward": (_ci, [_vp, _vp, _vp, _i64, _ci, _ci, _vp]),
    "tmb_softmax_backward_rows": (_ci, [_vp, _vp, _vp, _i64, _i64, _ci, _ci, _vp]),
    "tmb_nll_log_softmax_backward_rows": (_ci, [_vp] * 5 + [_i64] * 4 + [_ci, _i64, _ci, _vp]),
    "tmb_layer_norm_backward_workspace_bytes": (_sz, [_i64, _i64, _ci]),
    "tmb_layer_norm_backward_rows": (_ci, [_vp] * 8 + [_i64, _i64, _ci, _vp, _sz, _vp]),
    "tmb_layer_norm_backward_add_workspace_bytes": (_sz, [_i64, _i64, _ci]),
    "tmb_layer_norm_backward_add_rows": (_ci, [_vp] * 10 + [_i64, _i64, _ci, _vp, _sz, _vp]),
    "tmb_copy_bytes": (_ci, [_vp, _vp, _sz, _vp]),
    "tmb_read_bytes": (_ci, [_vp, _sz, _vp, _vp]),
    "tmb_cat2_rows": (_ci, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "tmb_reduce_cols_workspace_bytes": (_sz, [_i64, _i64, _ci]),
    "tmb_reduce_cols": (_ci, [_vp, _vp, _i64, _i64, _ci, _ci, _vp, _sz, _vp]),
    "tmb_pad_rows": (_ci, [_vp, _vp, _i64, _i64, _i64, _i64, _ci, _vp]),
}

_lib = None


class HipLibraryMissing(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """The loaded library; raises ``HipLibraryMissing`` (never falls back) when absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIBRARY_PATH):
            raise HipLibraryMissing(
                f"{LIBRARY_PATH} is not built. Build it with `sh {os.path.join(_CSRC, 'build.sh')}` "
                "(hipcc, gfx950). torch_mojo_backend has no CPU or PyTorch fallback for its hot ops."
            )
        handle = ctypes.CDLL(LIBRARY_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def status_string(code: int) -> str:
    return lib().tmb_status_string(int(code)).decode()
