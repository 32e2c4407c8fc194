"""Test helpers with the semantics of the reference's ``torch_mojo_backend/testing.py``:
``CallChecker`` proves that the backend's own implementation of an op ran (:32-136),
``check_functions_are_equivalent`` compares a function compiled with ``mojo_backend`` against
PyTorch eager on the same inputs (:139-166), ``check_outputs`` compares against PyTorch **CPU**
eager (:186-229) — the single yardstick of the reference's suite."""

from __future__ import annotations

from collections.abc import Callable
from dataclasses import dataclass

import torch

from torch_mojo_backend import mojo_backend


class CallChecker:
    """Asserts that at least one registered implementation was called.

    Registering the ``aten_functions`` twin of an op also accepts its ``aten_fast.fast_<name>``
    twin(s), so one test passes whether the op went through the graph surface or the eager
    surface."""

    def __init__(self):
        self._functions = None
        self._before = None

    @staticmethod
    def _fast_twins(func: Callable) -> list:
        name = getattr(func, "__name__", "")
        if not name.startswith("aten"):
            return []
        try:
            from torch_mojo_backend.eager_kernels import aten_fast
        except Exception:  # noqa: BLE001 - the eager surface is optional for graph-only tests
            return []
        base = f"fast_{name}"
        twins = []
        for attr in dir(aten_fast):
            if attr == base or attr.startswith(base + "_"):
                cand = getattr(aten_fast, attr)
                if hasattr(cand, "call_count"):
                    twins.append(cand)
        return twins

    def register(self, *funcs: Callable) -> None:
        expanded = []
        for f in funcs:
            if not hasattr(f, "call_count"):
                raise AssertionError(
                    f"{getattr(f, '__name__', f)} is not instrumented; set "
                    "TORCH_MOJO_BACKEND_TESTING=1 before importing torch_mojo_backend")
            expanded.append(f)
            expanded.extend(self._fast_twins(f))
        self._functions = expanded
        self._before = [f.call_count for f in expanded]

    def check_was_called(self) -> None:
        if self._functions is None:
            return
        if not any(f.call_count > b for f, b in zip(self._functions, self._before)):
            names = ", ".join(getattr(f, "__name__", str(f)) for f in self._functions)
            raise AssertionError(f"none of [{names}] was called")


@dataclass
class Conf:
    device: str
    compile: bool

    def __str__(self) -> str:
        return f"{self.device}, compile={self.compile}"


def _to_device(x, device):
    if isinstance(x, torch.Tensor):
        return x.to(device)
    if isinstance(x, (list, tuple)):
        return type(x)(_to_device(v, device) for v in x)
    return x


def _assert_same(got, want, rtol, atol):
    if isinstance(want, (list, tuple)):
        assert isinstance(got, (list, tuple)) and len(got) == len(want)
        for g, w in zip(got, want):
            _assert_same(g, w, rtol, atol)
        return
    if isinstance(want, torch.Tensor):
        assert isinstance(got, torch.Tensor), f"expected a tensor, got {type(got)}"
        assert got.shape == want.shape, f"shape {tuple(got.shape)} vs {tuple(want.shape)}"
        assert got.dtype == want.dtype, f"dtype {got.dtype} vs {want.dtype}"
        torch.testing.assert_close(got.cpu(), want.cpu(), rtol=rtol, atol=atol)
        return
    assert got == want


def check_functions_are_equivalent(fn: Callable, device: str, inputs: list, fn_compiled=None,
                                   rtol=None, atol=None):
    """``fn`` compiled with mojo_backend vs ``fn`` run eagerly, both on ``device``."""
    fn_compiled = fn_compiled or torch.compile(fn, backend=mojo_backend)
    inputs_on_device = [_to_device(x, device) for x in inputs]
    want = fn(*inputs_on_device)
    got = fn_compiled(*inputs_on_device)
    _assert_same(got, want, rtol, atol)


def check_outputs(fn: Callable, conf: Conf, inputs: list, rtol=None, atol=None):
    """``fn`` on ``conf.device`` (compiled with mojo_backend when ``conf.compile``) vs ``fn`` on
    CPU clones of the inputs: same device-independent shape/dtype, values within
    ``assert_close`` tolerances."""
    cpu_inputs = [_to_device(x, "cpu") for x in inputs]
    want = fn(*cpu_inputs)
    run = torch.compile(fn, backend=mojo_backend) if conf.compile else fn
    got = run(*[_to_device(x, conf.device) for x in inputs])
    _assert_same(got, want, rtol, atol)
