"""Helpers of the graph executor (error text, device discovery).

The error text keeps the reference's wording (torch_compile_backend/utils.py:21-49) because
users and tests match on it: the op's qualified name, the node index, "inputs of node were",
the issue-tracker URL and the user stack trace."""

from __future__ import annotations

from collections.abc import Callable

import torch


def get_accelerators() -> list:
    """HIP devices first, the CPU last — the ordering of the reference's ``get_accelerators``
    (utils.py:8-19). The CPU entry is kept for API compatibility (``len(...) - 1`` is how
    callers index it); no kernel of this package runs there."""
    result = [torch.device("cuda", i) for i in range(torch.cuda.device_count())]
    result.append(torch.device("cpu"))
    return result


def get_fully_qualified_name(func: Callable | str) -> str:
    """How an FX call target is named in error messages: ``module.qualname of type <type> `` for
    callables (aten overloads print as ``torch._ops.aten.<op>``-style names), ``torch.Tensor.<m>``
    for method names (reference utils.py:21-33; tests match on the op name inside)."""
    if isinstance(func, str):
        return "torch.Tensor." + func
    parts = [getattr(func, "__module__", None), getattr(func, "__qualname__", None)]
    module, qualname = parts
    name = (module + "." if module is not None else "") + (qualname if qualname is not None else "")
    return f"{name} of type {type(func)} "


def _describe(value) -> str:
    if isinstance(value, torch.Tensor):
        return f"Tensor(shape={tuple(value.shape)}, dtype={value.dtype}, device={value.device})"
    if isinstance(value, (list, tuple)):
        inner = ", ".join(_describe(v) for v in value)
        return f"[{inner}]" if isinstance(value, list) else f"({inner})"
    return repr(value)


def get_error_message(node: torch.fx.Node, node_idx: int, func_args, func_kwargs) -> str:
    if node.stack_trace is None:
        stack_trace = ("No stack trace available, likely because this node is the result of a "
                       "decomposition.")
    else:
        stack_trace = node.stack_trace
    kwargs_desc = {k: _describe(v) for k, v in func_kwargs.items()}
    return (
        f"Failing at node {node_idx} when executing function {get_fully_qualified_name(node.target)}. "
        f"inputs of node were: args={_describe(list(func_args))}, kwargs={kwargs_desc}. "
        f"You can open an issue at https://github.com/gabrieldemarmiesse/torch-mojo-backend/issues . "
        f"It comes from there in your code: \n"
        f"{stack_trace}\n"
    )
