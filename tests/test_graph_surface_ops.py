"""The graph-surface mapping functions of the hot ops, called the way the executor calls them
(MAPPING_TORCH_ATEN_TO_MOJO[op](*cuda tensors)) and through torch.compile(backend=mojo_backend),
against the oracle's ATen-level rules (oracle.aten_*, which follow aten_functions.py:681-785,
1002-1020, 2313-2320, 2556-2590, 3311-3346 of the reference) and PyTorch CPU eager."""

import math

import pytest
import torch

import oracle
from helpers import as64, assert_close64, seeded

pytestmark = pytest.mark.gpu
aten = torch.ops.aten


def _mapping(op):
    from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO
    return MAPPING_TORCH_ATEN_TO_MOJO[op]


def _compiled(fn):
    from torch_mojo_backend import mojo_backend
    return torch.compile(fn, backend=mojo_backend, fullgraph=True)


def _sum_bound(x, dims):
    """A-priori bound of a float32 tree sum: (n-1) 2^-24 sum|x| per output element."""
    n = math.prod(x.shape[d] for d in dims) if dims else x.numel()
    a = x.double().abs()
    s = a.sum(dim=dims) if dims else a.sum()
    return (max(n, 2) - 1) * 2.0 ** -24 * s.numpy()


REDUCE_CASES = [
    ((37, 513), None, False), ((37, 513), [], False), ((37, 513), [1], False), ((37, 513), [-1], True),
    ((37, 513), [0], False), ((5, 7, 65), [0, 2], True), ((5, 7, 65), [-2], False),
    ((5, 7, 65), [0, 1, 2], False), ((3, 200000), [1], False), ((1000,), None, True), ((), None, False),
]


@pytest.mark.parametrize("shape,dim,keepdim", REDUCE_CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["sum", "mean", "amax"])
def test_float_reductions_through_the_mapping(name, dtype, shape, dim, keepdim):
    x = seeded(shape, seed=len(shape) + 1, dtype=dtype)
    fn = _mapping(getattr(aten, name))
    call_dim = [] if (dim is None and name == "amax") else dim      # amax has no dim=None form
    got = fn(x.cuda(), call_dim, keepdim)
    want = getattr(oracle, "aten_" + name)(x, call_dim, keepdim)
    assert got.dtype == want.dtype == dtype and tuple(got.shape) == tuple(want.shape)
    if name == "amax":
        assert torch.equal(got.cpu(), want)                       # a maximum is exact
        return
    rank = len(shape)
    dims = sorted(d % rank for d in dim) if dim else list(range(rank))
    exact = x.double()
    exact = (exact.sum(dim=dims, keepdim=keepdim) if rank else exact)
    count = math.prod(shape[d] for d in dims) if rank else 1
    bound = _sum_bound(x, dims) if rank else 0.0
    if keepdim and rank:
        bound = bound.reshape(tuple(got.shape))
    if name == "mean":
        exact, bound = exact / count, bound / count
    assert_close64(got, exact.numpy(), extra_abs=bound, what=f"{name} {shape} dim={dim}")
    # and the oracle's own rounding of the same reduction sits within the same band
    assert_close64(got, as64(want), extra_abs=2 * bound, rounded_want=True, what="vs oracle")


@pytest.mark.parametrize("dtype", [torch.bool, torch.uint8, torch.int8, torch.int16, torch.int32,
                                   torch.int64])
@pytest.mark.parametrize("dim,keepdim", [(None, False), ([1], True), ([0, 1], False)])
def test_integer_sums_promote_to_int64_and_are_exact(dtype, dim, keepdim):
    g = torch.Generator().manual_seed(5)
    x = torch.randint(0, 2 if dtype == torch.bool else 100, (33, 1031), generator=g).to(dtype)
    got = _mapping(aten.sum)(x.cuda(), dim, keepdim)
    want = oracle.aten_sum(x, dim, keepdim)
    assert got.dtype == torch.int64 and torch.equal(got.cpu(), want)
    assert torch.equal(got.cpu(), torch.sum(x, dim=dim, keepdim=keepdim) if dim is not None
                       else torch.sum(x).reshape(want.shape))


def test_sum_and_mean_dtype_argument():
    x = seeded((19, 300), seed=3, dtype=torch.bfloat16)
    got = _mapping(aten.sum)(x.cuda(), [1], False, dtype=torch.float32)
    assert got.dtype == torch.float32
    assert_close64(got, x.double().sum(1).numpy(), extra_abs=_sum_bound(x, [1]))
    got = _mapping(aten.mean)(x.cuda(), [1], True, dtype=torch.float32)
    assert got.dtype == torch.float32 and got.shape == (19, 1)
    assert_close64(got, x.double().mean(1, keepdim=True).numpy(),
                   extra_abs=(_sum_bound(x, [1]) / 300).reshape(19, 1))
    ints = torch.arange(12).reshape(3, 4).to(torch.int32)
    got = _mapping(aten.sum)(ints.cuda(), None, False, dtype=torch.float32)
    assert got.dtype == torch.float32 and got.item() == 66.0
    with pytest.raises(TypeError, match="floating point"):
        _mapping(aten.mean)(ints.cuda())


def test_empty_inputs_follow_aten():
    e = torch.empty(0, 4)
    for dim, keepdim in ((None, False), ([0], False), ([0], True), ([1], False)):
        want = torch.sum(e, dim=dim, keepdim=keepdim) if dim is not None else torch.sum(e)
        got = _mapping(aten.sum)(e.cuda(), dim, keepdim)
        assert got.shape == want.shape and torch.equal(got.cpu(), want)
        assert torch.equal(oracle.aten_sum(e, dim, keepdim), want)
        want = torch.mean(e, dim=dim, keepdim=keepdim) if dim is not None else torch.mean(e)
        got = _mapping(aten.mean)(e.cuda(), dim, keepdim)
        assert got.shape == want.shape and torch.equal(got.cpu().isnan(), want.isnan())
    got = _mapping(aten.amax)(e.cuda(), [1], False)           # the result itself is empty
    assert got.shape == (0,)
    with pytest.raises(ValueError, match="non-zero size"):
        _mapping(aten.amax)(e.cuda(), [0], False)
    ints = torch.empty(3, 0, dtype=torch.int8)
    got = _mapping(aten.sum)(ints.cuda(), [1], False)
    assert got.dtype == torch.int64 and torch.equal(got.cpu(), torch.zeros(3, dtype=torch.int64))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("in_shape", [(64,), (7, 64), (3, 5, 64), (2, 3, 5, 64), (0, 64)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_linear_mapping_ranks_and_bias(dtype, tol, in_shape, with_bias):
    x = seeded(in_shape, seed=1, dtype=dtype)
    w = seeded((48, 64), seed=2, dtype=dtype)
    b = seeded((48,), seed=3, dtype=dtype) if with_bias else None
    got = _mapping(aten.linear)(x.cuda(), w.cuda(), None if b is None else b.cuda())
    want = oracle.aten_linear(x, w, b)
    assert got.dtype == dtype and tuple(got.shape) == tuple(want.shape) == in_shape[:-1] + (48,)
    if got.numel() == 0:
        return
    exact = x.double() @ w.double().t() + (0 if b is None else b.double())
    err = (got.double().cpu() - exact).norm() / exact.norm()
    assert err.item() <= tol
    assert_close64(got, as64(want), rtol=4 * tol, atol=4 * tol, rounded_want=True, what="vs oracle")


def test_linear_bias_is_added_in_fp32_before_the_one_cast():
    """matmul_ops.mojo:2651-2657: round(acc + bias), not round(round(acc) + bias). With
    acc = 256 + 1 (exactly representable in fp32, not in bf16) and bias = 1 the two differ."""
    x = torch.zeros(8, 64, dtype=torch.bfloat16)
    x[:, 0], x[:, 1] = 16.0, 1.0
    w = torch.zeros(16, 64, dtype=torch.bfloat16)
    w[:, 0], w[:, 1] = 16.0, 1.0                                       # acc = 257
    b = torch.ones(16, dtype=torch.bfloat16)
    got = _mapping(aten.linear)(x.cuda(), w.cuda(), b.cuda()).float().cpu()
    assert torch.all(got == 258.0)                                     # bf16(258) = 258; bf16(257)+1 -> 256+1 -> 256 or 258
    twice = (torch.tensor(257.0).bfloat16().float() + 1.0).bfloat16().float()
    assert twice.item() != 258.0                                       # the wrong order is visible here


SOFTMAX_SHAPES = [((33, 257), -1), ((4, 6, 50), 1), ((4, 6, 50), 0), ((5, 1000), -2), ((9,), 0), ((), -1)]


@pytest.mark.parametrize("shape,dim", SOFTMAX_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_softmax_dtype_argument_and_dims(shape, dim, dtype):
    x = seeded(shape, seed=7, scale=4.0, dtype=dtype)
    for arg in (None, torch.float32):
        got = _mapping(aten.softmax)(x.cuda(), dim, arg)
        out_dtype = arg or dtype
        assert got.dtype == out_dtype and got.shape == x.shape
        src = x.double()
        want = torch.softmax(src, dim) if x.dim() else torch.ones((), dtype=torch.float64)
        assert_close64(got, want.numpy(), what=f"softmax {shape} dim={dim} dtype={arg}")
    # half_to_float on the underscore op: the oracle's rule
    if dtype != torch.float32 and x.dim():
        got = _mapping(aten._softmax)(x.cuda(), dim, True)
        want = oracle.aten__softmax(x, dim, True)
        assert got.dtype == torch.float32
        assert_close64(got, as64(want), rounded_want=True)


@pytest.mark.parametrize("shape,dim", SOFTMAX_SHAPES)
def test_log_softmax_half_to_float_rule(shape, dim):
    x16 = seeded(shape, seed=8, scale=4.0, dtype=torch.float16)
    got = _mapping(aten._log_softmax)(x16.cuda(), dim, True)
    assert got.dtype == torch.float32
    want = torch.log_softmax(x16.double(), dim) if x16.dim() else torch.zeros((), dtype=torch.float64)
    assert_close64(got, want.numpy(), atol=2e-6)
    assert_close64(got, as64(oracle.aten__log_softmax(x16, dim, True)), atol=4e-6, rounded_want=True)
    xb = x16.to(torch.bfloat16)
    with pytest.raises(ValueError, match="Half"):
        _mapping(aten._log_softmax)(xb.cuda(), dim, True)
    got = _mapping(aten._log_softmax)(xb.cuda(), dim, False)
    assert got.dtype == torch.bfloat16


def test_the_same_rules_through_torch_compile():
    """One compiled function per rule: the executor must reach the same mapping functions
    (call counts) and return what the direct calls return."""
    from torch_mojo_backend import aten_functions as af

    x = seeded((37, 513), seed=11, dtype=torch.bfloat16)
    ints = torch.randint(0, 50, (12, 77), generator=torch.Generator().manual_seed(1)).to(torch.int32)
    w = seeded((48, 513), seed=12, dtype=torch.bfloat16)
    b = seeded((48,), seed=13, dtype=torch.bfloat16)

    def fn(x, ints, w, b):
        return (torch.sum(x, dim=1), torch.sum(ints), torch.sum(ints, dim=0, keepdim=True),
                torch.mean(x, dim=[0, 1]), torch.mean(x, dim=-1, keepdim=True, dtype=torch.float32),
                torch.amax(x, dim=[0]), torch.amax(x),
                torch.softmax(x, dim=-1, dtype=torch.float32), torch.log_softmax(x, dim=0),
                torch.nn.functional.linear(x, w, b))

    before = {f.__name__: f.call_count for f in (af.aten_sum, af.aten_mean, af.aten_amax)}
    with torch.no_grad():
        got = _compiled(fn)(x.cuda(), ints.cuda(), w.cuda(), b.cuda())
    assert af.aten_sum.call_count - before["aten_sum"] == 3
    assert af.aten_mean.call_count - before["aten_mean"] == 2
    assert af.aten_amax.call_count - before["aten_amax"] == 2
    want = fn(x, ints, w, b)
    assert [g.dtype for g in got] == [t.dtype for t in want]
    assert [tuple(g.shape) for g in got] == [tuple(t.shape) for t in want]
    assert torch.equal(got[1].cpu(), want[1]) and torch.equal(got[2].cpu(), want[2])
    assert torch.equal(got[5].cpu(), want[5]) and torch.equal(got[6].cpu(), want[6])
    assert_close64(got[0], x.double().sum(1).numpy(), extra_abs=_sum_bound(x, [1]))
    assert_close64(got[3], x.double().mean().numpy(), extra_abs=_sum_bound(x, [0, 1]) / x.numel())
    assert_close64(got[4], x.double().mean(-1, keepdim=True).numpy(),
                   extra_abs=(_sum_bound(x, [1]) / 513).reshape(37, 1))
    assert_close64(got[7], torch.softmax(x.double(), -1).numpy())
    assert_close64(got[8], torch.log_softmax(x.double(), 0).numpy(), atol=2e-6)
    exact = x.double() @ w.double().t() + b.double()
    assert ((got[9].double().cpu() - exact).norm() / exact.norm()).item() <= 1e-2
