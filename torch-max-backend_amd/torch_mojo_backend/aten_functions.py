"""The aten -> kernel registry of the ``mojo_backend`` graph surface.

Mirrors the contract of the reference's ``torch_mojo_backend/aten_functions.py``:

* ``MAPPING_TORCH_ATEN_TO_MOJO`` (reference :116) is a plain mutable dict keyed by
  ``OpOverload`` / ``OpOverloadPacket`` / python builtins; users may add, override or delete
  entries at run time;
* ``map_to(op)`` (reference :157-198) registers a function, counts its calls under
  ``TORCH_MOJO_BACKEND_TESTING=1`` and removes the op (every overload of a packet) from
  ``DECOMPOSITION_TABLE`` (reference :113) so AOTAutograd hands the op over undecomposed;
* mapping functions take the ATen schema's arguments. Here the tensors are real
  ``torch.Tensor``s on a HIP device instead of MAX graph values, and a mapping function
  *executes* its op.

The hot ops (mm / addmm / bmm / linear, _softmax / softmax / _log_softmax, native_layer_norm,
sum / mean / amax / argmax, gelu) run on the hand-written gfx950 kernels of ``libtmb_hip.so``.
Every other op the reference maps is registered as the PyTorch-ROCm op itself, so whole
models run with ``fullgraph=True``; those are not part of this package's kernel layer.
"""

from __future__ import annotations

import contextvars
import functools
import operator
import os
from typing import List, Optional

import math

import torch
from torch._decomp import core_aten_decompositions
from torch._ops import OpOverload, OpOverloadPacket

import torch_mojo_backend.is_running_tests
from torch_mojo_backend import eager_kernels as _ek
from torch_mojo_backend.eager_kernels import hip_ops
from torch_mojo_backend.flags import verbose_enabled

aten = torch.ops.aten

# The fx node currently executed, set by the graph executor; lets multi-output mappings see
# which outputs are consumed (reference :98-109).
CURRENT_FX_NODE: contextvars.ContextVar = contextvars.ContextVar("CURRENT_FX_NODE", default=None)


def _only_first_output_used() -> bool:
    node = CURRENT_FX_NODE.get()
    if node is None:
        return False
    return all(user.target is operator.getitem and user.args[1] == 0 for user in node.users)


DECOMPOSITION_TABLE = core_aten_decompositions()
original_decomposition_table_size = len(DECOMPOSITION_TABLE)
MAPPING_TORCH_ATEN_TO_MOJO: dict = {}

IDENTICAL_FUNCTIONS = [
    operator.add, operator.sub, operator.mul, operator.truediv, operator.floordiv, operator.pow,
    operator.mod, operator.matmul, operator.neg, operator.gt, operator.ge, operator.lt,
    operator.le, operator.eq, operator.ne, operator.and_, operator.or_, operator.xor,
    operator.iadd, operator.isub, operator.imul, operator.ifloordiv, operator.ipow,
    operator.imod, operator.getitem, str, max, min,
]
for _func in IDENTICAL_FUNCTIONS:
    MAPPING_TORCH_ATEN_TO_MOJO[_func] = _func

number_of_decompositions_removed = 0


def map_to(func):
    """Register the decorated function as the implementation of ``func``."""

    def decorator(func_to_map):
        global number_of_decompositions_removed
        if os.environ.get("TORCH_MOJO_BACKEND_BEARTYPE", "0") == "1":
            try:
                from beartype import beartype
            except ImportError:  # optional dependency
                beartype = None
            if beartype is not None:
                func_to_map = beartype(func_to_map)

        registered = func_to_map
        if torch_mojo_backend.is_running_tests.IS_RUNNING_TESTS:

            @functools.wraps(func_to_map)
            def counted(*args, **kwargs):
                counted.call_count += 1
                return func_to_map(*args, **kwargs)

            counted.call_count = 0
            registered = counted

        if isinstance(func, OpOverload):
            DECOMPOSITION_TABLE.pop(func, None)
        elif isinstance(func, OpOverloadPacket):
            for overload_name in func.overloads():
                if DECOMPOSITION_TABLE.pop(getattr(func, overload_name), None) is not None:
                    number_of_decompositions_removed += 1
        else:
            raise TypeError(f"Expected OpOverload or OpOverloadPacket, got {type(func)}")
        MAPPING_TORCH_ATEN_TO_MOJO[func] = registered
        return registered

    return decorator


# ---------------------------------------------------------------------------
# Hot ops on the HIP kernels
# ---------------------------------------------------------------------------
def _normalize_dims(dim, rank: int) -> List[int]:
    """None / [] -> all dims; ints wrapped; sorted (reference :1002-1020, :3311-3346)."""
    if dim is None:
        return list(range(rank))
    if isinstance(dim, int):
        dim = [dim]
    dims = [d % rank if rank else 0 for d in dim]
    if not dims:
        return list(range(rank))
    if len(set(dims)) != len(dims):
        raise ValueError(f"dim {tuple(dim)} has duplicates")
    return sorted(dims)


@map_to(aten.mm)
def aten_mm(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """reference :2632-2634."""
    return hip_ops.gemm(x, y)


@map_to(aten.bmm)
def aten_bmm(input: torch.Tensor, mat2: torch.Tensor) -> torch.Tensor:
    """reference :1415-1428."""
    return hip_ops.gemm(input, mat2)


@map_to(aten.addmm)
def aten_addmm(input: torch.Tensor, mat1: torch.Tensor, mat2: torch.Tensor, *, beta=1.0,
               alpha=1.0) -> torch.Tensor:
    """``beta*input + alpha*(mat1 @ mat2)`` (reference :971-992). A ``[n]`` bias with
    beta == alpha == 1 is fused into the GEMM epilogue (added in fp32 before the one cast,
    matmul_ops.mojo:2651-2657); any other case scales and adds afterwards."""
    n = mat2.shape[-1]
    if beta == 1 and alpha == 1 and input.dim() == 1 and input.shape[0] == n \
            and input.dtype == mat1.dtype:
        return hip_ops.gemm(mat1, mat2, input)
    result = hip_ops.gemm(mat1, mat2)
    if alpha != 1:
        result = result * alpha
    scaled = input * beta if beta != 1 else input
    return scaled + result


def addmm_gelu(input: torch.Tensor, mat1: torch.Tensor, mat2: torch.Tensor,
               approximate: str = "none", round_like_unfused: bool = False) -> torch.Tensor:
    """``gelu(addmm(bias, mat1, mat2))`` in one kernel. Produced by the executor's
    addmm -> view -> gelu fusion. The GELU works on the float32 sum and the result is cast once
    (the reference forms what it fuses into a GEMM in float32 and casts once,
    matmul_ops.mojo:2651-2657); with ``round_like_unfused`` the sum is rounded to the storage
    dtype first, which makes the result bit-identical to the unfused pair."""
    epi = _ek.EPI_GELU_TANH if approximate == "tanh" else _ek.EPI_GELU_ERF
    return hip_ops.gemm(mat1, mat2, input, epilogue=epi, round_like_unfused=round_like_unfused)


def addmm_residual(input: torch.Tensor, mat1: torch.Tensor, mat2: torch.Tensor,
                   residual: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                   round_like_unfused: bool = False) -> torch.Tensor:
    """``addmm(bias, mat1, mat2) + residual`` in one kernel (residual reshaped to the product's
    [M, N]). Produced by the executor's addmm -> view -> add fusion. Summed in float32 and cast
    once; ``residual`` and the result may be float32 for 16-bit operands (the residual stream of a
    16-bit graph kept in float32). With ``round_like_unfused`` the product is rounded to the
    storage dtype before the add: the bits of the unfused pair."""
    m, n = mat1.shape[0], mat2.shape[-1]
    return hip_ops.gemm(mat1, mat2, input, residual=residual.reshape(m, n), out_dtype=out_dtype,
                        round_like_unfused=round_like_unfused)


@map_to(aten.linear)
def aten_linear(input: torch.Tensor, weight: torch.Tensor,
                bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``input @ weight.T + bias`` (reference :2313-2320); the weight is read K-major in place."""
    lead = input.shape[:-1]
    x2 = input.reshape(-1, input.shape[-1]) if input.dim() != 2 else input
    out = hip_ops.gemm(x2, weight.t(), bias)
    return out if input.dim() == 2 else out.reshape(*lead, weight.shape[0])


@map_to(aten._softmax)
def aten__softmax(self: torch.Tensor, dim: int, half_to_float: bool) -> torch.Tensor:
    """reference :681-687."""
    return hip_ops.softmax(self, dim, half_to_float=half_to_float)


@map_to(aten.softmax)
def aten_softmax(input: torch.Tensor, dim: int = -1, dtype=None) -> torch.Tensor:
    """reference :690-714: an explicit dtype casts the input first."""
    if dtype is not None and dtype != input.dtype:
        if dtype == torch.float32 and input.dtype in (torch.float16, torch.bfloat16):
            return hip_ops.softmax(input, dim, half_to_float=True)
        input = input.to(dtype)
    return hip_ops.softmax(input, dim)


@map_to(aten._log_softmax)
def aten__log_softmax(input: torch.Tensor, dim: int, half_to_float: bool) -> torch.Tensor:
    """reference :718-785: half_to_float is float16-only."""
    if half_to_float and input.dtype != torch.float16:
        raise ValueError(
            f"half_to_float conversion is supported for Half (float16) type only, got {input.dtype}")
    return hip_ops.softmax(input, dim, half_to_float=half_to_float, log=True)


@map_to(aten.native_layer_norm)
def aten_native_layer_norm(input: torch.Tensor, normalized_shape, weight: Optional[torch.Tensor],
                           bias: Optional[torch.Tensor], eps: float):
    """(out, mean, rstd) with keepdim float32 statistics (reference :2829-2868). When only
    output 0 is consumed the statistics are neither allocated nor written (reference
    :2837-2849)."""
    normalized_shape = [int(s) for s in normalized_shape]
    if _only_first_output_used():
        out, _, _ = hip_ops.layer_norm(input, normalized_shape, weight, bias, eps, need_stats=False)
        return out, None, None
    return hip_ops.layer_norm(input, normalized_shape, weight, bias, eps)


_INT_PROMOTE = (torch.bool, torch.uint8, torch.int8, torch.int16, torch.int32)


def _reduced_shape(shape, dims, keepdim: bool) -> List[int]:
    if keepdim:
        return [1 if d in dims else s for d, s in enumerate(shape)]
    return [s for d, s in enumerate(shape) if d not in dims]


@map_to(aten.sum)
def aten_sum(input: torch.Tensor, dim=None, keepdim: bool = False, *, dtype=None) -> torch.Tensor:
    """reference :3311-3346: small integer / bool inputs are summed as int64; an empty reduction
    is 0 (eager twin: aten_fast.py:3033-3037)."""
    if dtype is not None:
        input = input.to(dtype)
    elif input.dtype in _INT_PROMOTE:
        input = input.to(torch.int64)
    dims = _normalize_dims(dim, input.dim())
    if input.numel() == 0:
        return torch.zeros(_reduced_shape(input.shape, dims, keepdim), dtype=input.dtype,
                           device=input.device)
    return hip_ops.reduce(input, dims, keepdim, _ek.SUM)


@map_to(aten.mean)
def aten_mean(input: torch.Tensor, dim=None, keepdim: bool = False, *, dtype=None) -> torch.Tensor:
    """reference :2556-2590. The mean of no elements is NaN (0/0), as in ATen."""
    if dtype is not None:
        input = input.to(dtype)
    if not input.dtype.is_floating_point:
        raise TypeError(f"mean(): could not infer output dtype. Input dtype must be floating point, "
                        f"got {input.dtype}")
    dims = _normalize_dims(dim, input.dim())
    if input.numel() == 0:
        return torch.full(_reduced_shape(input.shape, dims, keepdim), float("nan"),
                          dtype=input.dtype, device=input.device)
    return hip_ops.reduce(input, dims, keepdim, _ek.MEAN)


@map_to(aten.amax)
def aten_amax(input: torch.Tensor, dim=[], keepdim: bool = False) -> torch.Tensor:
    """reference :1002-1020. A maximum over no elements does not exist: ValueError, unless the
    result itself is empty."""
    dims = _normalize_dims(dim, input.dim())
    if input.numel() == 0:
        if any(input.shape[d] == 0 for d in dims):
            raise ValueError(f"amax(): expected every reduced dim of {tuple(input.shape)} to have "
                             f"non-zero size, got dims {dims}")
        return torch.empty(_reduced_shape(input.shape, dims, keepdim), dtype=input.dtype,
                           device=input.device)
    return hip_ops.reduce(input, dims, keepdim, _ek.AMAX)


@map_to(aten.argmax)
def aten_argmax(input: torch.Tensor, dim: Optional[int] = None, keepdim: bool = False) -> torch.Tensor:
    """reference :1141-1196."""
    return hip_ops.argmax(input, dim, keepdim)


@map_to(aten.embedding)
def aten_embedding(weight: torch.Tensor, indices: torch.Tensor, padding_idx: int = -1,
                   scale_grad_by_freq: bool = False, sparse: bool = False) -> torch.Tensor:
    """reference :1780-1795 (the remaining arguments only matter to the backward)."""
    if weight.dim() == 2 and weight.dtype in hip_ops.FLOAT_DTYPES and weight.shape[0] > 0 \
            and indices.dtype in (torch.int32, torch.int64):
        return hip_ops.embedding(weight, indices)
    return torch.ops.aten.embedding(weight, indices, padding_idx, scale_grad_by_freq, sparse)


@map_to(aten.gelu)
def aten_gelu(input: torch.Tensor, approximate: str = "none") -> torch.Tensor:
    """reference :2063-2067."""
    return hip_ops.gelu(input, approximate)


@map_to(aten.scaled_dot_product_attention)
def aten_scaled_dot_product_attention(query, key, value, attn_mask=None, dropout_p: float = 0.0,
                                      is_causal: bool = False, *, scale=None,
                                      enable_gqa: bool = False) -> torch.Tensor:
    """reference :3029-3087 (built there from matmul, softmax and matmul graph ops). The fused
    HIP kernel takes the call when there is no explicit mask, head_dim is 64 and the dtype has
    16 bits; up to 16 queries per head (decode) run in the decode kernel; other head sizes, fp32
    and additive masks run as GEMM + softmax + GEMM on the same kernels. Dropout and grouped-query attention are PyTorch-ROCm's own op."""
    plain = dropout_p == 0.0 and not enable_gqa and query.dim() >= 2 \
        and query.dtype in hip_ops.FLOAT_DTYPES and key.dtype == query.dtype \
        and value.dtype == query.dtype and key.shape[:-2] == query.shape[:-2] \
        and value.shape[:-2] == query.shape[:-2] and query.numel() > 0 and key.shape[-2] > 0 \
        and not (attn_mask is not None and is_causal)
    if plain:
        s = float(scale) if scale is not None else 1.0 / math.sqrt(query.shape[-1])
        if query.dim() == 4 and query.shape[2] <= hip_ops.DECODE_MAX_QUERIES \
                and hip_ops.attention_decode_supported(query, key, value, attn_mask):
            return hip_ops.attention_decode(query, key, value, s, bool(is_causal), attn_mask)
        if attn_mask is None and s > 0.0 and query.dim() == 4 \
                and hip_ops.attention_supported(query, key, value):
            return hip_ops.attention(query, key, value, s, bool(is_causal)).transpose(1, 2)
        return hip_ops.attention_composed(query, key, value, s, bool(is_causal), attn_mask)
    return aten.scaled_dot_product_attention(query, key, value, attn_mask, dropout_p, is_causal,
                                             scale=scale, enable_gqa=enable_gqa)


_FLASH_EXTRAS: dict = {}


def _flash_extras(like: torch.Tensor) -> tuple:
    """The outputs of aten::_scaled_dot_product_flash_attention that carry nothing without
    dropout: the two random-number-state scalars (int64 on ROCm) and the empty debug mask.
    Nothing ever writes them, so one set per (device, dtype) serves every call."""
    key = (like.device, like.dtype)
    if key not in _FLASH_EXTRAS:
        _FLASH_EXTRAS[key] = (torch.zeros((), dtype=torch.int64, device=like.device),
                              torch.zeros((), dtype=torch.int64, device=like.device),
                              torch.empty(0, dtype=like.dtype, device=like.device))
    return _FLASH_EXTRAS[key]


def _flash_scale(query, scale) -> float:
    return float(scale) if scale is not None else 1.0 / math.sqrt(query.shape[-1])


@map_to(aten._scaled_dot_product_flash_attention)
def aten__scaled_dot_product_flash_attention(query, key, value, dropout_p: float = 0.0,
                                             is_causal: bool = False,
                                             return_debug_mask: bool = False, *, scale=None):
    """reference :540-677 (which returns a zero log-sum-exp: "we don't support training yet") and
    eager_kernels/aten_fast.py:4211-4248 (which returns the real one). What torch.compile makes of
    F.scaled_dot_product_attention on 16-bit CUDA tensors: output laid out like the query, the
    float32 log-sum-exp the backward op needs, and the placeholders of the 9-value contract.
    Dropout, a debug mask, other head sizes: PyTorch-ROCm's own op."""
    s = _flash_scale(query, scale)
    if dropout_p == 0.0 and not return_debug_mask and query.dim() == 4 and s > 0.0 \
            and hip_ops.attention_supported(query, key, value):
        out, lse = hip_ops.attention(query, key, value, s, bool(is_causal), return_lse=True,
                                     like_query=True)
        seed, offset, debug_mask = _flash_extras(query)
        return (out, lse, None, None, query.shape[2], key.shape[2], seed, offset, debug_mask)
    return aten._scaled_dot_product_flash_attention(query, key, value, dropout_p, is_causal,
                                                    return_debug_mask, scale=scale)


@map_to(aten._scaled_dot_product_flash_attention_backward)
def aten__scaled_dot_product_flash_attention_backward(grad_out, query, key, value, out, logsumexp,
                                                      cum_seq_q, cum_seq_k, max_q, max_k,
                                                      dropout_p, is_causal, philox_seed,
                                                      philox_offset, *, scale=None):
    """eager_kernels/aten_fast.py:4251-4338 (the graph surface of the reference has no attention
    backward). (grad_query, grad_key, grad_value), each laid out like its input."""
    s = _flash_scale(query, scale)
    if dropout_p == 0.0 and cum_seq_q is None and cum_seq_k is None and s > 0.0 \
            and query.dim() == 4 and logsumexp.is_contiguous() \
            and hip_ops.attention_backward_supported(grad_out, query, key, value, out, logsumexp):
        return hip_ops.attention_backward(grad_out, query, key, value, out, logsumexp, s,
                                          bool(is_causal))
    return aten._scaled_dot_product_flash_attention_backward(
        grad_out, query, key, value, out, logsumexp, cum_seq_q, cum_seq_k, max_q, max_k,
        dropout_p, is_causal, philox_seed, philox_offset, scale=scale)


# ---------------------------------------------------------------------------
# Backward twins of the hot ops (reference :788-833, :2070-2102, :2323-2375; the layer-norm
# backward is eager-only there, eager_kernels/aten_fast.py:2797-2913)
# ---------------------------------------------------------------------------
@map_to(aten.gelu_backward)
def aten_gelu_backward(grad_output: torch.Tensor, input: torch.Tensor, *,
                       approximate: str = "none") -> torch.Tensor:
    if approximate not in ("none", "tanh"):
        raise ValueError(f"Invalid approximate argument '{approximate}'. Supported values are "
                         "'none' and 'tanh'.")
    return hip_ops.gelu_backward(grad_output, input, approximate)


def _softmax_backward(grad_output, output, dim, input_dtype, log):
    if grad_output.dtype != output.dtype:
        raise ValueError("grad_output and output must have the same dtype")
    if tuple(grad_output.shape) != tuple(output.shape):
        raise ValueError("grad_output and output must have the same shape")
    if grad_output.dtype != input_dtype and not (
            grad_output.dtype == torch.float32 and input_dtype == torch.float16):
        raise ValueError("input and grad dtypes must match, or input must be float16 and grad "
                         "must be float32")
    rank = grad_output.dim()
    if rank and not -rank <= dim < rank:
        raise ValueError("dim must refer to an input dimension")
    if rank == 0 and dim not in (-1, 0):
        raise ValueError("dim must be -1 or 0 for a scalar input")
    result = hip_ops.softmax_backward(grad_output, output, dim, log)
    return result if result.dtype == input_dtype else result.to(input_dtype)


@map_to(aten._log_softmax_backward_data)
def aten__log_softmax_backward_data(grad_output: torch.Tensor, output: torch.Tensor, dim: int,
                                    input_dtype: torch.dtype) -> torch.Tensor:
    """reference :788-833: grad - exp(output) * sum(grad, dim)."""
    return _softmax_backward(grad_output, output, dim, input_dtype, True)


@map_to(aten._softmax_backward_data)
def aten__softmax_backward_data(grad_output: torch.Tensor, output: torch.Tensor, dim: int,
                                input_dtype: torch.dtype) -> torch.Tensor:
    """output * (grad - sum(grad * output, dim)): the same row kernel in its softmax form."""
    return _softmax_backward(grad_output, output, dim, input_dtype, False)


@map_to(aten.native_layer_norm_backward)
def aten_native_layer_norm_backward(grad_out, input, normalized_shape, mean, rstd, weight, bias,
                                    output_mask):
    """(grad_input, grad_weight, grad_bias) from the saved statistics (eager twin:
    aten_fast.py:2797-2913)."""
    mask = [bool(m) for m in output_mask]
    if len(mask) != 3:
        raise ValueError("native_layer_norm_backward output_mask must contain three booleans")
    if (mask[1] and weight is None) or (mask[2] and bias is None):
        raise ValueError("native_layer_norm_backward: a parameter gradient was requested for a "
                         "parameter that is None")
    return hip_ops.layer_norm_backward(grad_out, input, normalized_shape, mean.float(),
                                       rstd.float(), weight, mask)


@map_to(aten.linear_backward)
def aten_linear_backward(self, grad_output, weight, output_mask):
    """reference :2323-2375."""
    mask = tuple(output_mask)
    if len(mask) != 3 or any(not isinstance(m, bool) for m in mask):
        raise ValueError("linear_backward output_mask must contain three booleans")
    if self.dim() < 1 or weight.dim() != 2:
        raise ValueError("linear_backward expects rank >= 1 input and rank 2 weight")
    return hip_ops.linear_backward(self, grad_output, weight, mask)


HOT_OPS = (aten.mm, aten.bmm, aten.addmm, aten.linear, aten._softmax, aten.softmax,
           aten._log_softmax, aten.native_layer_norm, aten.sum, aten.mean, aten.amax,
           aten.argmax, aten.gelu)

# ---------------------------------------------------------------------------
# Every other op the reference maps: the PyTorch-ROCm op itself.
# ---------------------------------------------------------------------------
_PASSTHROUGH = """
floordiv _local_scalar_dense all _adaptive_avg_pool2d _adaptive_avg_pool2d_backward
_native_batch_norm_legit_no_training _scaled_dot_product_attention_math
_scaled_dot_product_efficient_attention
_to_copy abs acos add addcdiv addcmul alias amin any arange
argmin asinh atanh avg_pool2d bitwise_and.Scalar bitwise_and.Tensor bitwise_not bitwise_or.Scalar
bitwise_or.Tensor bitwise_xor.Scalar bitwise_xor.Tensor cat ceil clamp clone constant_pad_nd
convolution copy cos cosh cumsum detach div empty.memory_format empty_strided empty_like
empty_permuted eq erf exp expand fill fill_ floor full full_like ge gt index isin
isnan le lift_fresh_copy log log1p logical_and logical_not logical_xor lt
max max_pool2d_with_indices maximum mean.out min minimum mul native_batch_norm native_group_norm
normal_ ne neg nonzero ones_like permute pow reciprocal relu remainder repeat relu_ rsqrt
scalar_tensor scaled_dot_product_attention scatter.src scatter.value select select_scatter sigmoid
sign silu sin tan tanh sinh slice split_with_sizes sqrt squeeze sub unsqueeze upsample_bilinear2d
var view _unsafe_view where stack tril triu split unbind t.default _foreach_add.Scalar
_foreach_add.ScalarList _foreach_add.Tensor _foreach_add.List _foreach_sub.Scalar
_foreach_sub.ScalarList _foreach_sub.List _foreach_mul.Scalar _foreach_mul.ScalarList
_foreach_mul.Tensor _foreach_mul.List _foreach_neg _foreach_pow.Scalar _foreach_pow.ScalarList
_foreach_pow.List _foreach_pow.ScalarAndTensor _foreach_div.Scalar _foreach_div.ScalarList
_foreach_div.Tensor _foreach_div.List _foreach_reciprocal _foreach_sqrt _foreach_addcdiv.Scalar
_foreach_addcdiv.ScalarList _foreach_addcmul.Scalar _foreach_addcmul.ScalarList masked_fill
transpose sym_size sym_numel sym_stride sym_storage_offset
""".split()

# Cold ops that only a backward graph contains (loss, embedding and indexing gradients): beyond
# what the reference's graph surface maps, so that a compiled training step runs end to end.
_PASSTHROUGH += """
index_put index_put_ gather scatter_add nll_loss_forward nll_loss_backward nll_loss2d_forward
embedding_dense_backward tanh_backward sigmoid_backward threshold_backward new_zeros new_empty
new_empty_strided zeros_like zeros ones sum_to_size expand_as squeeze_ unsqueeze_ mse_loss
mse_loss_backward _softmax_backward_data.out log sqrt_ rsub addcmul_ addcdiv_ lerp
_scaled_dot_product_efficient_attention_backward
""".split()


def _resolve(name: str):
    obj = aten
    for part in name.split("."):
        obj = getattr(obj, part, None)
        if obj is None:
            return None
    return obj


def _passthrough(op):
    def run(*args, **kwargs):
        return op(*args, **kwargs)

    run.__name__ = "aten_" + str(getattr(op, "__name__", op)).replace(".", "_")
    run.__qualname__ = run.__name__
    return run


for _name in _PASSTHROUGH:
    _op = _resolve(_name)
    if _op is not None and _op not in MAPPING_TORCH_ATEN_TO_MOJO:
        map_to(_op)(_passthrough(_op))

if verbose_enabled():
    print(f"Removed {number_of_decompositions_removed}/{original_decomposition_table_size} decompositions.")
