"""Pins for the CPU oracle (no GPU needed).

Every oracle function is checked against things that do not share its code: float64 closed
forms, brute-force Python loops on tiny inputs, library routines (scipy), mathematical
invariants, PyTorch CPU eager (the yardstick of the reference's own tests,
torch_mojo_backend/testing.py:186-229) and the committed fixtures in tests/golden/.
Each block is built so that a plausible slip (dropped term, transposed operand, unbiased
instead of biased variance, bias added after the cast, last instead of first index) fails it.
"""

import math
import os

import numpy as np
import pytest
import scipy.special
import torch

import oracle
from oracle import closed_form as cf
from helpers import as64, assert_close64, seeded

FLOATS = [torch.float32, torch.bfloat16, torch.float16]


# ---------------------------------------------------------------------------
# 16-bit conversions of the C oracle vs PyTorch's
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,code", [(torch.bfloat16, oracle.BF16), (torch.float16, oracle.F16)])
def test_conversions_match_torch_bit_for_bit(dtype, code):
    L = oracle.lib()
    # every 16-bit pattern -> float32
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    out = torch.empty(65536, dtype=torch.float32)
    L.orc_convert_to_f32(out.data_ptr(), bits.data_ptr(), 65536, code)
    want = bits.view(dtype).float()
    isnan = torch.isnan(want)  # signalling-NaN payloads may be quieted differently; NaN-ness must agree
    assert torch.equal(torch.isnan(out), isnan)
    assert torch.equal(out.view(torch.int32)[~isnan], want.view(torch.int32)[~isnan])
    # float32 -> 16 bit: random values, exact ties, subnormals, overflow, inf, nan
    g = torch.Generator().manual_seed(0)
    vals = torch.cat([
        torch.randn(200000, generator=g) * 10 ** torch.randint(-8, 6, (200000,), generator=g).float(),
        want[torch.isfinite(want)],                                  # representable values
        (want[:-1] + want[1:])[torch.isfinite(want[:-1] + want[1:])] / 2,  # midpoints (ties)
        torch.tensor([0.0, -0.0, float("inf"), float("-inf"), float("nan"), 65504.0, 65519.9,
                      65520.0, 65536.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 3.4e38, -3.4e38]),
    ])
    got = torch.empty(vals.numel(), dtype=torch.int16)
    L.orc_convert_from_f32(got.data_ptr(), vals.data_ptr(), vals.numel(), code)
    ref = vals.to(dtype).view(torch.int16)
    nan = torch.isnan(vals)
    assert torch.equal(got[~nan], ref[~nan])
    assert torch.isnan(got[nan].view(dtype).float()).all()


# ---------------------------------------------------------------------------
# GEMM
# ---------------------------------------------------------------------------
def _brute_gemm(a, b, bias):
    m, k = a.shape
    n = b.shape[1]
    out = [[0.0] * n for _ in range(m)]
    for i in range(m):
        for j in range(n):
            acc = 0.0
            for kk in range(k):
                acc += float(a[i, kk]) * float(b[kk, j])
            out[i][j] = acc + (float(bias[j]) if bias is not None else 0.0)
    return np.array(out)


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("mnk", [(1, 1, 1), (2, 3, 4), (5, 2, 7), (4, 6, 3)])
def test_gemm_brute_force(mnk, dtype):
    m, n, k = mnk
    a, b, bias = seeded((m, k), 1, dtype=dtype), seeded((k, n), 2, dtype=dtype), seeded((n,), 3, dtype=dtype)
    want = _brute_gemm(a.double().numpy(), b.double().numpy(), bias.double().numpy())
    assert_close64(oracle.gemm(a, b, bias), want, what="gemm brute")
    assert_close64(oracle.gemm(a, b), want - bias.double().numpy(), what="gemm no bias")
    # the same product through transposed / strided views (operands are NOT symmetric)
    bt = b.t().contiguous().t()
    assert torch.equal(oracle.gemm(a, bt, bias), oracle.gemm(a, b, bias))
    at = a.t().contiguous().t()
    assert torch.equal(oracle.gemm(at, b, bias), oracle.gemm(a, b, bias))


@pytest.mark.parametrize("dtype", FLOATS)
def test_gemm_vs_closed_form_and_torch(dtype):
    a, b, bias = seeded((37, 129), 4, dtype=dtype), seeded((129, 53), 5, dtype=dtype), seeded((53,), 6, dtype=dtype)
    want = cf.gemm(as64(a), as64(b), as64(bias))
    bound = 129 * 2.0 ** -24 * (np.abs(as64(a)) @ np.abs(as64(b)) + np.abs(as64(bias)))
    got = oracle.aten_addmm(bias, a, b)
    assert_close64(got, want, extra_abs=bound, what="addmm closed form")
    torch.testing.assert_close(got, torch.addmm(bias, a, b))
    torch.testing.assert_close(oracle.aten_mm(a, b), torch.mm(a, b))
    w = seeded((53, 129), 7, dtype=dtype)
    x3 = seeded((2, 5, 129), 8, dtype=dtype)
    torch.testing.assert_close(oracle.aten_linear(x3, w, bias), torch.nn.functional.linear(x3, w, bias))
    a3, b3 = seeded((3, 9, 17), 9, dtype=dtype), seeded((3, 17, 11), 10, dtype=dtype)
    torch.testing.assert_close(oracle.aten_bmm(a3, b3), torch.bmm(a3, b3))
    torch.testing.assert_close(oracle.aten_bmm(a3, b3.transpose(1, 2).contiguous().transpose(1, 2)),
                               torch.bmm(a3, b3))
    # alpha / beta and a full-matrix input take the unfused route
    inp = seeded((37, 53), 11, dtype=dtype)
    torch.testing.assert_close(oracle.aten_addmm(inp, a, b, beta=0.5, alpha=2.0),
                               torch.addmm(inp, a, b, beta=0.5, alpha=2.0), rtol=2e-2, atol=2e-2)


def test_gemm_bias_is_added_in_fp32_before_the_cast():
    a = torch.zeros(1, 2, dtype=torch.bfloat16)
    b = torch.zeros(2, 1, dtype=torch.bfloat16)
    a[0, 0], b[0, 0], a[0, 1], b[1, 0] = 1.0, 1.0, 2.0 ** -8, 1.0
    bias = torch.tensor([2.0 ** -10], dtype=torch.bfloat16)
    fused = oracle.gemm(a, b, bias)
    assert fused.item() == 1.0 + 2.0 ** -7                       # one rounding of 1+2^-8+2^-10
    assert (oracle.gemm(a, b) + bias).item() == 1.0              # two roundings would give 1.0


@pytest.mark.parametrize("dtype", FLOATS)
def test_gemm_gelu_epilogue_both_rounding_modes(dtype):
    a, b, bias = seeded((9, 16), 1, dtype=dtype), seeded((16, 12), 2, dtype=dtype), seeded((12,), 3, dtype=dtype)
    pre = oracle.gemm(a, b, bias)
    exact = as64(a) @ as64(b) + as64(bias)
    for epi, approx in ((oracle.EPI_GELU_TANH, "tanh"), (oracle.EPI_GELU_ERF, "none")):
        # like the unfused pair: gelu of the sum as a separate addmm kernel would have stored it
        twice = oracle.gemm(a, b, bias, epilogue=epi, round_like_unfused=True)
        assert torch.equal(twice, oracle.gelu(pre, approx))
        torch.testing.assert_close(twice, torch.nn.functional.gelu(pre, approximate=approx))
        # default: gelu of the float32 sum, one cast -> the correctly rounded gelu of the exact sum
        once = oracle.gemm(a, b, bias, epilogue=epi)
        want = torch.nn.functional.gelu(torch.from_numpy(exact), approximate=approx).numpy()
        assert_close64(once, want, what=f"gelu({approx}) of the fp32 sum")
    if dtype != torch.float32:
        # a case where the two differ: acc + bias = 1 + 2^-9 is no bf16/fp16-tie-free number
        a1 = torch.tensor([[1.0, 2.0 ** -9 if dtype == torch.bfloat16 else 2.0 ** -12]], dtype=dtype)
        b1 = torch.ones(2, 1, dtype=dtype)
        z = torch.zeros(1, dtype=dtype)
        x = a1.double().sum().item()
        once = oracle.gemm(a1, b1, z, epilogue=oracle.EPI_GELU_ERF).double().item()
        twice = oracle.gemm(a1, b1, z, epilogue=oracle.EPI_GELU_ERF, round_like_unfused=True).double().item()
        g = lambda v: 0.5 * v * (1 + math.erf(v / math.sqrt(2)))  # noqa: E731
        assert once == torch.tensor(g(x), dtype=torch.float64).to(dtype).double().item()
        assert twice == torch.tensor(g(1.0), dtype=torch.float64).to(dtype).double().item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gemm_residual_rounding_modes_and_float32_stream(dtype):
    a, b = seeded((7, 24), 4, dtype=dtype), seeded((24, 10), 5, dtype=dtype)
    bias = seeded((10,), 6, dtype=dtype)
    r32 = seeded((7, 10), 7, scale=3.0)
    r16 = r32.to(dtype)
    exact = as64(a) @ as64(b) + as64(bias)
    # float32 residual in, float32 out: nothing is rounded to 16 bits anywhere
    wide = oracle.gemm(a, b, bias, residual=r32, out_dtype=torch.float32)
    assert wide.dtype == torch.float32
    np.testing.assert_allclose(as64(wide), exact + as64(r32), rtol=1e-6, atol=1e-6)
    # float32 residual in, 16-bit out; 16-bit residual in, float32 out; 16-bit both: one rounding
    assert_close64(oracle.gemm(a, b, bias, residual=r32), exact + as64(r32), what="f32 residual")
    np.testing.assert_allclose(as64(oracle.gemm(a, b, bias, residual=r16, out_dtype=torch.float32)),
                               exact + as64(r16), rtol=1e-6, atol=1e-6)
    once = oracle.gemm(a, b, bias, residual=r16)
    assert_close64(once, exact + as64(r16), what="one rounding")
    # like the unfused pair: PyTorch CPU's addmm (fp32 accumulate, one cast) followed by add
    twice = oracle.gemm(a, b, bias, residual=r16, round_like_unfused=True)
    assert torch.equal(twice, oracle.gemm(a, b, bias) + r16)
    torch.testing.assert_close(twice, torch.addmm(bias, a, b) + r16)
    # the two orders are told apart: the product 1 + eps (half a spacing of the storage type at 1)
    # rounds to 1 before the residual eps is added in the unfused order; in float32 the sum
    # 1 + 2 eps is exact and representable
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    a1, b1 = torch.tensor([[1.0, eps]], dtype=dtype), torch.ones(2, 1, dtype=dtype)
    res = torch.tensor([[eps]], dtype=dtype)
    assert oracle.gemm(a1, b1, None, residual=res).double().item() == 1.0 + 2 * eps
    assert oracle.gemm(a1, b1, None, residual=res, round_like_unfused=True).double().item() == 1.0
    # batched, and a transposed operand
    a3, b3 = seeded((3, 5, 8), 8, dtype=dtype), seeded((3, 6, 8), 9, dtype=dtype).transpose(1, 2)
    rr = seeded((3, 5, 6), 10)
    got = oracle.gemm(a3, b3, None, residual=rr, out_dtype=torch.float32)
    np.testing.assert_allclose(as64(got), np.einsum("bmk,bkn->bmn", as64(a3), as64(b3)) + as64(rr),
                               rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_layer_norm_float32_rows_into_16_bit_output(out_dtype):
    x = seeded((6, 200), 11, scale=2.0, shift=0.5)
    g = seeded((200,), 12, scale=0.1, shift=1.0, dtype=out_dtype)
    b = seeded((200,), 13, scale=0.1, dtype=out_dtype)
    out, mean, rstd = oracle.layer_norm_rows(x, g, b, 1e-5, out_dtype=out_dtype)
    assert out.dtype == out_dtype and mean.dtype == torch.float32
    w_out, w_mean, w_rstd = cf.layer_norm(as64(x), as64(g), as64(b), 1e-5)
    scale = np.abs(as64(x) - w_mean) * w_rstd * np.abs(as64(g)) + np.abs(as64(b))
    assert_close64(out, w_out, extra_abs=1e-5 * scale)
    assert_close64(mean.reshape(-1, 1), w_mean, atol=1e-6)
    assert_close64(rstd.reshape(-1, 1), w_rstd, rtol=1e-5)
    # the statistics come from the float32 values, not from values rounded to the output type
    rounded, m16, _ = oracle.layer_norm_rows(x.to(out_dtype), g, b, 1e-5)
    assert not torch.equal(m16, mean)
    same, m32, _ = oracle.layer_norm_rows(x, g.float(), b.float(), 1e-5)
    assert torch.equal(m32, mean) and torch.equal(same.to(out_dtype), out)


# ---------------------------------------------------------------------------
# softmax / log_softmax
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", [(1, 1), (3, 2), (5, 33), (4, 257), (2, 5000)])
def test_softmax_closed_form_library_and_invariants(shape, dtype):
    x = seeded(shape, shape[1], scale=4.0, dtype=dtype)
    got = oracle.softmax_rows(x)
    assert_close64(got, cf.softmax(as64(x)), what="softmax closed form")
    assert_close64(got, scipy.special.softmax(as64(x), axis=-1), what="softmax scipy")
    torch.testing.assert_close(got, torch.softmax(x, -1))
    lg = oracle.softmax_rows(x, log=True)
    assert_close64(lg, scipy.special.log_softmax(as64(x), axis=-1), what="log_softmax scipy")
    # PyTorch's 16-bit CPU log_softmax is itself only good to a storage ulp of the row maximum
    loose = {torch.float32: {}, torch.bfloat16: dict(rtol=2e-2, atol=4e-2),
             torch.float16: dict(rtol=2e-3, atol=4e-3)}[dtype]
    torch.testing.assert_close(lg, torch.log_softmax(x, -1), **loose)
    if dtype == torch.float32:
        # the reference kernel sums the denominator sequentially in fp32: n*2^-24 a priori
        assert np.abs(as64(got).sum(-1) - 1).max() < max(2e-6, shape[1] * 2.0 ** -24)
        shifted = oracle.softmax_rows(x + 5.0)
        assert_close64(shifted, as64(got), rtol=1e-5 + shape[1] * 2.0 ** -24, atol=1e-7, what="shift invariance")
        assert np.abs(np.exp(as64(lg)).sum(-1) - 1).max() < 1e-5 + shape[1] * 2.0 ** -24


def test_softmax_brute_force_and_extremes():
    x = torch.tensor([[0.5, -1.25, 3.0], [1000.0, 999.0, -1000.0]])
    want = []
    for row in x.tolist():
        m = max(row)
        e = [math.exp(v - m) for v in row]
        want.append([v / sum(e) for v in e])
    assert_close64(oracle.softmax_rows(x), np.array(want), what="brute")
    assert torch.isnan(oracle.softmax_rows(torch.tensor([[1.0, float("nan"), 2.0]]))).all()
    out = oracle.softmax_rows(torch.tensor([[float("-inf"), 0.0, 0.0]]))
    assert out.tolist() == [[0.0, 0.5, 0.5]]


@pytest.mark.parametrize("dim", [0, 1, 2, -1, -2])
def test_aten_softmax_dims_and_half_to_float(dim):
    x = seeded((4, 5, 6), 3, scale=2.0)
    torch.testing.assert_close(oracle.aten__softmax(x, dim, False), torch.softmax(x, dim))
    torch.testing.assert_close(oracle.aten__log_softmax(x, dim, False), torch.log_softmax(x, dim))
    h = x.to(torch.float16)
    out = oracle.aten__softmax(h, dim, True)
    assert out.dtype == torch.float32
    torch.testing.assert_close(out, torch.softmax(h.float(), dim))
    assert oracle.aten__log_softmax(h, dim, True).dtype == torch.float32
    with pytest.raises(ValueError, match="Half"):
        oracle.aten__log_softmax(x.bfloat16(), dim, True)
    assert oracle.aten__softmax(torch.tensor(2.0), -1, False).item() == 1.0
    assert oracle.aten__log_softmax(torch.tensor(2.0), -1, False).item() == 0.0


# ---------------------------------------------------------------------------
# layer norm
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", [(1, 2), (3, 7), (5, 65), (4, 768), (2, 4097)])
def test_layer_norm_closed_form_and_torch(shape, dtype):
    rows, cols = shape
    x = seeded(shape, cols, scale=2.0, shift=0.3, dtype=dtype)
    g, b = seeded((cols,), 1, scale=0.1, shift=1.0, dtype=dtype), seeded((cols,), 2, scale=0.1, dtype=dtype)
    out, mean, rstd = oracle.aten_native_layer_norm(x, [cols], g, b, 1e-5)
    assert mean.dtype == torch.float32 and tuple(mean.shape) == (rows, 1)
    w_out, w_mean, w_rstd = cf.layer_norm(as64(x), as64(g), as64(b), 1e-5)
    scale = np.abs(as64(x) - w_mean) * w_rstd * np.abs(as64(g)) + np.abs(as64(b))
    assert_close64(out, w_out, extra_abs=2e-5 * scale, what="ln out")
    assert_close64(mean, w_mean, rtol=1e-5, atol=2e-6, what="ln mean")
    assert_close64(rstd, w_rstd, rtol=2e-5, what="ln rstd")
    t_out, t_mean, t_rstd = torch.native_layer_norm(x, [cols], g, b, 1e-5)
    torch.testing.assert_close(out, t_out)
    # PyTorch CPU returns the statistics of a 16-bit input rounded to that 16-bit type; the
    # reference compares them at 2e-2 in that case (tests/test_eager_kernels.py:525-541)
    st = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(mean, t_mean.float(), **st)
    st = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(rstd, t_rstd.float(), **st)


def test_layer_norm_brute_force_biased_variance_and_shapes():
    x = torch.tensor([[1.0, 2.0, 3.0, 6.0]])
    out, mean, rstd = oracle.layer_norm_rows(x, None, None, 0.0)
    mu = 3.0
    var = ((1 - mu) ** 2 + (2 - mu) ** 2 + 0 + (6 - mu) ** 2) / 4          # biased: /n, not /(n-1)
    assert mean.item() == mu and abs(rstd.item() - 1 / math.sqrt(var)) < 1e-7
    assert_close64(out, np.array([[(v - mu) / math.sqrt(var) for v in (1, 2, 3, 6)]]), what="brute")
    # eps enters inside the square root
    _, _, rstd2 = oracle.layer_norm_rows(x, None, None, 0.5)
    assert abs(rstd2.item() - 1 / math.sqrt(var + 0.5)) < 1e-7
    # multi-dim normalized_shape: keepdim float32 statistics
    x3 = seeded((2, 3, 4), 5)
    w, b = seeded((3, 4), 6), seeded((3, 4), 7)
    got = oracle.aten_native_layer_norm(x3, (3, 4), w, b, 0.5)
    want = torch.native_layer_norm(x3, (3, 4), w, b, 0.5)
    assert tuple(got[1].shape) == (2, 1, 1)
    for a_, b_ in zip(got, want):
        torch.testing.assert_close(a_, b_, rtol=1e-5, atol=1e-5)
    # gamma=1, beta=0 => zero mean / unit variance
    y, _, _ = oracle.layer_norm_rows(seeded((16, 768), 8, scale=3.0, shift=1.0), None, None, 1e-5)
    assert y.double().mean(-1).abs().max() < 1e-6
    assert (y.double().var(-1, unbiased=False) - 1).abs().max() < 1e-4


@pytest.mark.parametrize("value", [float("nan"), float("inf"), float("-inf")])
def test_layer_norm_nonfinite_rows_are_nan(value):
    x = torch.full((2, 9), value)
    out, mean, rstd = oracle.layer_norm_rows(x, None, None, 1e-5)
    assert torch.isnan(out).all() and torch.isnan(mean).all() and torch.isnan(rstd).all()


# ---------------------------------------------------------------------------
# reductions and argmax
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (7, 1000), (2, 65537)])
def test_reduce_rows_vs_float64(shape, dtype):
    x = seeded(shape, shape[1] % 13, dtype=dtype)
    x64 = as64(x)
    bound = cf.sum_error_bound(x64)
    assert_close64(oracle.reduce_rows(x, oracle.SUM), x64.sum(-1), extra_abs=bound, what="sum")
    assert_close64(oracle.reduce_rows(x, oracle.MEAN), x64.mean(-1), extra_abs=bound / shape[1], what="mean")
    assert np.array_equal(as64(oracle.reduce_rows(x, oracle.AMAX)), x64.max(-1))
    tiny = torch.tensor([[1.0, 2.0, 4.0], [-1.0, -8.0, -3.0]], dtype=dtype)
    assert oracle.reduce_rows(tiny, oracle.SUM).tolist() == [7.0, -12.0]
    assert oracle.reduce_rows(tiny, oracle.MEAN).tolist() == [pytest.approx(7 / 3, rel=1e-2), -4.0]
    assert oracle.reduce_rows(tiny, oracle.AMAX).tolist() == [4.0, -1.0]


@pytest.mark.parametrize("dim,keepdim", [(None, False), ([], False), (0, False), ([1], True),
                                         ([0, 2], False), ([-1], True), ([0, 1, 2], True)])
def test_aten_reductions_follow_torch(dim, keepdim):
    x = seeded((4, 5, 6), 2)
    tdim = None if dim in (None, []) else dim
    torch.testing.assert_close(oracle.aten_sum(x, dim, keepdim), torch.sum(x, dim=tdim, keepdim=keepdim)
                               if tdim is not None else (x.sum().reshape([1, 1, 1]) if keepdim else x.sum()))
    torch.testing.assert_close(oracle.aten_mean(x, dim, keepdim), torch.mean(x, dim=tdim, keepdim=keepdim)
                               if tdim is not None else (x.mean().reshape([1, 1, 1]) if keepdim else x.mean()))
    adim = [] if dim is None else dim
    torch.testing.assert_close(oracle.aten_amax(x, adim, keepdim), torch.amax(x, dim=adim, keepdim=keepdim))


def test_aten_sum_integer_promotion_and_empty():
    for dt in (torch.bool, torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64):
        x = (seeded((3, 50), 1) * 10).to(dt)
        got = oracle.aten_sum(x, [1])
        assert got.dtype == torch.int64 and torch.equal(got, x.sum(1))
    big = torch.full((2, 3), 2 ** 40, dtype=torch.int64)
    assert oracle.aten_sum(big).item() == 6 * 2 ** 40
    assert oracle.aten_amax(big * torch.tensor([[1], [-1]]), [1]).tolist() == [2 ** 40, -2 ** 40]
    assert oracle.aten_sum(torch.zeros(0, 4), [0]).tolist() == [0.0] * 4
    assert oracle.aten_sum(seeded((2, 3), 1).bfloat16(), dtype=torch.float32).dtype == torch.float32


@pytest.mark.parametrize("dtype", FLOATS + [torch.int64, torch.int32])
def test_argmax_first_occurrence(dtype):
    x = (seeded((50, 300), 3) * 100).to(dtype)
    x[:, 200] = x[:, 100] = x.max() if dtype.is_floating_point else int(x.max())  # tie: 100 wins
    got = oracle.argmax_rows(x)
    assert (got == 100).all()
    brute = [max(range(300), key=lambda j, r=r: (float(x[r, j]), -j)) for r in range(50)]
    assert got.tolist() == brute
    y = (seeded((20, 1001), 4) * 100).to(dtype)
    assert torch.equal(oracle.argmax_rows(y), torch.argmax(y, dim=1))
    assert torch.equal(oracle.argmax_rows(y), torch.from_numpy(cf.argmax_first(y.double().numpy())))


def test_argmax_nan_and_aten_dims():
    x = seeded((3, 10), 1)
    x[0, 4] = x[0, 7] = float("nan")
    x[1, 0] = float("nan")
    assert oracle.argmax_rows(x).tolist()[:2] == [4, 0]
    assert torch.equal(oracle.argmax_rows(x), torch.argmax(x, dim=1))
    z = seeded((4, 5, 6), 5)
    assert torch.equal(oracle.aten_argmax(z), torch.argmax(z))
    assert oracle.aten_argmax(z, None, True).shape == (1, 1, 1)
    for d in (0, 1, 2, -1, -3):
        for keep in (False, True):
            assert torch.equal(oracle.aten_argmax(z, d, keep), torch.argmax(z, dim=d, keepdim=keep))


# ---------------------------------------------------------------------------
# GELU
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", FLOATS)
def test_gelu_closed_forms(dtype):
    x = seeded((4000,), 1, scale=3.0, dtype=dtype)
    assert_close64(oracle.gelu(x, "tanh"), cf.gelu_tanh(as64(x)), atol=2e-6, what="gelu tanh")
    assert_close64(oracle.gelu(x, "none"), cf.gelu_erf(as64(x)), atol=2e-6, what="gelu erf")
    torch.testing.assert_close(oracle.gelu(x, "tanh"), torch.nn.functional.gelu(x, approximate="tanh"))
    torch.testing.assert_close(oracle.gelu(x, "none"), torch.nn.functional.gelu(x))
    pts = torch.tensor([0.0, 1.0, -1.0, 10.0, -10.0])
    want = [0.5 * v * (1 + math.erf(v / math.sqrt(2))) for v in pts.tolist()]
    assert_close64(oracle.gelu(pts, "none"), np.array(want), atol=1e-7, what="gelu points")


# ---------------------------------------------------------------------------
# committed fixtures (PyTorch CPU eager outputs, see tests/golden/make_fixtures.py)
# ---------------------------------------------------------------------------
def _golden():
    path = os.path.join(os.path.dirname(__file__), "golden", "hot_ops_torch_cpu.npz")
    return np.load(path, allow_pickle=False)


def _t(arr, dtype_name):
    t = torch.from_numpy(np.ascontiguousarray(arr))
    if dtype_name == "bfloat16":
        return t.view(torch.bfloat16)
    return t


def test_oracle_reproduces_golden_fixtures():
    g = _golden()
    # softmax [33,257] fp32 (x4 scaled)
    torch.testing.assert_close(oracle.softmax_rows(_t(g["softmax_x"], "float32")), _t(g["softmax_y"], "float32"))
    torch.testing.assert_close(oracle.softmax_rows(_t(g["softmax_x"], "float32"), log=True),
                               _t(g["log_softmax_y"], "float32"))
    # layer norm [3,65] bf16 triple
    x, w, b = (_t(g[k], "bfloat16") for k in ("ln_x", "ln_w", "ln_b"))
    out, mean, rstd = oracle.aten_native_layer_norm(x, [65], w, b, 1e-5)
    torch.testing.assert_close(out, _t(g["ln_out"], "bfloat16"))
    torch.testing.assert_close(mean, _t(g["ln_mean"], "float32"), rtol=2e-2, atol=2e-2)  # bf16-rounded
    torch.testing.assert_close(rstd, _t(g["ln_rstd"], "float32"), rtol=2e-2, atol=2e-2)  # by PyTorch
    # argmax with ties [4,50257]
    assert torch.equal(oracle.argmax_rows(_t(g["argmax_x"], "float32")), _t(g["argmax_y"], "int64"))
    # addmm bf16 [17,24]x[24,40]
    a, bm, bias = (_t(g[k], "bfloat16") for k in ("mm_a", "mm_b", "mm_bias"))
    torch.testing.assert_close(oracle.aten_addmm(bias, a, bm), _t(g["mm_out"], "bfloat16"))
    # sums
    sx = _t(g["sum_x"], "float32")
    torch.testing.assert_close(oracle.aten_sum(sx, [1]), _t(g["sum_rows"], "float32"), rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(oracle.aten_amax(sx, [1]), _t(g["amax_rows"], "float32"), rtol=0, atol=0)


# ---------------------------------------------------------------- attention softmax (scale, causal)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
def test_softmax_scaled_closed_form_and_invariants(dtype, causal):
    x = seeded((3, 2, 37, 37), seed=21, scale=3.0, dtype=dtype)
    scale = 0.125
    got = oracle.softmax_scaled(x, scale, causal_q_len=37 if causal else 0)
    want = cf.softmax_scaled_causal(as64(x), scale, causal)
    tol = {torch.float32: 2e-6, torch.bfloat16: 4e-3, torch.float16: 5e-4}[dtype]
    assert np.abs(as64(got) - want).max() <= tol
    np.testing.assert_allclose(as64(got).sum(-1), 1.0, atol=37 * tol)
    if causal:
        upper = np.triu(np.ones((37, 37), dtype=bool), 1)
        assert (as64(got)[..., upper] == 0).all()          # exact zeros above the diagonal
        assert (as64(got)[..., 0, 0] == 1.0).all()          # first query row sees one key


def test_softmax_scaled_reduces_to_plain_softmax_and_to_torch_pipeline():
    x = seeded((5, 64, 64), seed=22, scale=2.0, dtype=torch.bfloat16)
    # scale 1, no mask: the very same arithmetic as orc_softmax
    assert torch.equal(oracle.softmax_scaled(x, 1.0), oracle.softmax_rows(x.reshape(-1, 64)).reshape(x.shape))
    # rounded product + causal mask == what PyTorch's three separate ops compute (bf16 storage
    # between them); torch's CPU softmax rounds once from fp32 as well
    mask = torch.tril(torch.ones(64, 64)) == 0
    want = torch.softmax((x * 0.3).masked_fill(mask, float("-inf")), dim=-1)
    got = oracle.softmax_scaled(x, 0.3, causal_q_len=64, round_scaled=True)
    assert np.abs(as64(got) - as64(want)).max() <= 2 ** -8
    # without the rounding the result differs from it only by the bf16 rounding of the product
    free = oracle.softmax_scaled(x, 0.3, causal_q_len=64, round_scaled=False)
    assert np.abs(as64(free) - as64(got)).max() <= 3e-2


def test_softmax_scaled_brute_force_tiny():
    x = torch.tensor([[[1.0, 2.0, 3.0], [0.5, -1.0, 4.0], [2.0, 2.0, 2.0]]])
    got = as64(oracle.softmax_scaled(x, 2.0, causal_q_len=3))
    rows = []
    for r in range(3):
        e = [math.exp(2.0 * x[0, r, j].item()) if j <= r else 0.0 for j in range(3)]
        rows.append([v / sum(e) for v in e])
    np.testing.assert_allclose(got[0], np.array(rows), rtol=1e-6)


# ---------------------------------------------------------------- attention (unfused chain)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [False, True])
def test_attention_oracle_vs_closed_form_and_torch(dtype, causal):
    q = seeded((2, 3, 33, 16), seed=41, dtype=dtype)
    k = seeded((2, 3, 33, 16), seed=42, dtype=dtype)
    v = seeded((2, 3, 33, 16), seed=43, dtype=dtype)
    got = oracle.attention(q, k, v, 0.25, causal)
    assert got.shape == (2, 33, 3, 16)
    want = cf.attention(as64(q), as64(k), as64(v), 0.25, causal)
    tol = {torch.float32: 5e-6, torch.bfloat16: 3e-2, torch.float16: 4e-3}[dtype]
    assert np.abs(as64(got) - want).max() <= tol
    # PyTorch's own fused op on the CPU, same inputs (what the reference's tests compare with)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(),
                                                           is_causal=causal, scale=0.25)
    assert np.abs(as64(got) - as64(ref.transpose(1, 2))).max() <= tol


def test_attention_oracle_special_cases():
    # one key: the output is that key's value row, whatever the scores
    q = seeded((1, 2, 5, 8), seed=1)
    k = seeded((1, 2, 1, 8), seed=2)
    v = seeded((1, 2, 1, 8), seed=3)
    got = oracle.attention(q, k, v, 3.0, False)
    np.testing.assert_allclose(as64(got), np.broadcast_to(as64(v).transpose(0, 2, 1, 3), (1, 5, 2, 8)), rtol=1e-6)
    # causal: query 0 sees only key 0
    k2, v2 = seeded((1, 2, 5, 8), seed=4), seeded((1, 2, 5, 8), seed=5)
    got2 = oracle.attention(q, k2, v2, 1.0, True)
    np.testing.assert_allclose(as64(got2)[:, 0], as64(v2)[:, :, 0], rtol=1e-6)
    # identical keys: uniform weights -> the mean of the values
    k3 = torch.ones(1, 1, 4, 8)
    v3 = seeded((1, 1, 4, 8), seed=6)
    got3 = oracle.attention(seeded((1, 1, 2, 8), seed=7), k3, v3, 1.0, False)
    np.testing.assert_allclose(as64(got3)[0, :, 0], np.broadcast_to(as64(v3)[0, 0].mean(0), (2, 8)), rtol=1e-6)


# ---------------------------------------------------------------- backward twins
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("approximate", ["none", "tanh"])
def test_gelu_backward_oracle_vs_autograd_and_limits(dtype, approximate):
    x = (seeded((9, 77), seed=1) * 3).to(dtype)
    g = seeded((9, 77), seed=2).to(dtype)
    got = oracle.gelu_backward(g, x, approximate)
    x64 = x.double().requires_grad_(True)
    (torch.nn.functional.gelu(x64, approximate=approximate) * g.double()).sum().backward()
    tol = {torch.float32: 1e-6, torch.bfloat16: 2e-2, torch.float16: 3e-3}[dtype]
    assert (got.double() - x64.grad).abs().max().item() <= tol * 5
    # gelu'(0) = 1/2, gelu'(+large) = 1, gelu'(-large) = 0
    pts = torch.tensor([0.0, 40.0, -40.0], dtype=dtype)
    lim = oracle.gelu_backward(torch.full_like(pts, 2.0), pts, approximate).float()
    assert torch.allclose(lim, torch.tensor([1.0, 2.0, 0.0]), atol=1e-6)


@pytest.mark.parametrize("reduction", ["none", "mean", "sum"])
def test_nll_log_softmax_backward_oracle_vs_autograd(reduction):
    """The oracle's loss backward against float64 autograd of `nll_loss(log_softmax(x))`, with
    ignored rows, for every reduction; and by brute force on a tiny case."""
    torch.manual_seed(5)
    x = torch.randn(9, 37, dtype=torch.float64, requires_grad=True)
    t = torch.randint(0, 37, (9,))
    t[3], t[7] = -100, -100
    logp = torch.log_softmax(x, 1)
    loss = torch.nn.functional.nll_loss(logp, t, reduction=reduction)
    up = torch.rand(9, dtype=torch.float64) + 0.5 if reduction == "none" else torch.tensor(1.25, dtype=torch.float64)
    loss.backward(up)
    code = {"none": 0, "mean": 1, "sum": 2}[reduction]
    got = oracle.nll_log_softmax_backward(up.float(), logp.detach().float(), t, torch.tensor(7.0), code, -100)
    torch.testing.assert_close(got.double(), x.grad, rtol=1e-5, atol=1e-6)
    assert float(got[3].abs().max()) == 0.0 and float(got[7].abs().max()) == 0.0
    # brute force: w * (exp(logp) - [c == t])
    lp = logp.detach().float()
    for r in (0, 4):
        w = float(up[r]) if reduction == "none" else float(up) / (7.0 if reduction == "mean" else 1.0)
        for c in (0, int(t[r]), 36):
            want = w * (float(torch.exp(lp[r, c])) - (1.0 if c == int(t[r]) else 0.0))
            assert abs(float(got[r, c]) - want) <= 1e-6
    # a target that is no class behaves like an ignored one (the reference kernel's rule)
    t2 = t.clone()
    t2[0] = 37
    got2 = oracle.nll_log_softmax_backward(up.float(), lp, t2, torch.tensor(7.0), code, -100)
    assert float(got2[0].abs().max()) == 0.0


@pytest.mark.parametrize("log", [False, True])
def test_softmax_backward_oracle_vs_autograd_and_invariants(log):
    x = seeded((7, 130), seed=3)
    g = seeded((7, 130), seed=4)
    xr = x.double().requires_grad_(True)
    out = (torch.log_softmax if log else torch.softmax)(xr, -1)
    (out * g.double()).sum().backward()
    got = oracle.softmax_backward_rows(g, out.detach().float(), log)
    assert (got.double() - xr.grad).abs().max().item() <= 5e-6
    # brute force on a tiny row from the Jacobian d out_i / d x_j
    y = torch.softmax(torch.tensor([[0.3, -1.2, 2.0]]), -1)
    gg = torch.tensor([[1.0, -2.0, 0.5]])
    if log:
        jac = torch.eye(3) - y.expand(3, 3)            # d log y_i / d x_j = delta_ij - y_j
        saved = y.log()
    else:
        jac = torch.diag(y[0]) - y.t() @ y             # d y_i / d x_j = y_i (delta_ij - y_j)
        saved = y
    want = gg @ jac
    torch.testing.assert_close(oracle.softmax_backward_rows(gg, saved, log), want, rtol=1e-5, atol=1e-6)
    # a gradient that is constant along the row: zero for softmax; rows sum to zero for log-softmax
    const = oracle.softmax_backward_rows(torch.full((7, 130), 2.5), out.detach().float(), log)
    if log:
        assert const.sum(-1).abs().max().item() <= 1e-4
    else:
        assert const.abs().max().item() <= 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("affine", [True, False])
def test_layer_norm_backward_oracle_vs_autograd_and_invariants(dtype, affine):
    rows, cols = 11, 96
    x = seeded((rows, cols), seed=5).to(dtype)
    g = seeded((rows, cols), seed=6).to(dtype)
    w = (1 + 0.1 * seeded((cols,), seed=7)).to(dtype) if affine else None
    _, mean, rstd = oracle.layer_norm_rows(x, w, None, 1e-5)
    dx, dw, db = oracle.layer_norm_backward_rows(g, x, mean, rstd, w)
    x64 = x.double().requires_grad_(True)
    w64 = None if w is None else w.double().requires_grad_(True)
    b64 = torch.zeros(cols, dtype=torch.float64, requires_grad=True)
    (torch.nn.functional.layer_norm(x64, [cols], w64, b64, 1e-5) * g.double()).sum().backward()
    tol = {torch.float32: 2e-5, torch.bfloat16: 4e-2}[dtype]
    assert (dx.double() - x64.grad).abs().max().item() <= tol * 4
    assert (db.double() - b64.grad).abs().max().item() <= tol * 8
    if affine:
        assert (dw.double() - w64.grad).abs().max().item() <= tol * 8
    if dtype == torch.float32:
        # grad_input is orthogonal to the constant vector and to xhat (the two directions the
        # normalisation removes); grad_bias is the column sum of the upstream gradient
        xhat = (x - mean.view(-1, 1)) * rstd.view(-1, 1)
        assert dx.sum(-1).abs().max().item() <= 1e-4
        assert (dx * xhat).sum(-1).abs().max().item() <= 1e-3
        torch.testing.assert_close(db, g.sum(0), rtol=1e-5, atol=1e-5)


# --- attention backward -------------------------------------------------------------------------
def _attention_math_f64(q, k, v, scale, causal):
    """float64 autograd chain: the definition the oracle's backward is pinned to."""
    s = (q @ k.transpose(-1, -2)) * scale
    if causal:
        t, n = s.shape[-2:]
        s = s.masked_fill(torch.ones(t, n, dtype=torch.bool).triu(1), float("-inf"))
    return torch.softmax(s, -1) @ v, torch.logsumexp(s, -1)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 1, 1, 1, 4), (2, 3, 7, 7, 8), (1, 2, 5, 9, 16)])
def test_attention_lse_and_backward_match_float64_autograd(shape, causal):
    b, h, t, s_len, d = shape
    g = torch.Generator().manual_seed(sum(shape) + causal)
    q, k, v = (torch.randn(b, h, n, d, generator=g) for n in (t, s_len, s_len))
    dout = torch.randn(b, t, h, d, generator=g)
    scale = 0.37
    q64, k64, v64 = (x.double().requires_grad_(True) for x in (q, k, v))
    out64, lse64 = _attention_math_f64(q64, k64, v64, scale, causal)
    out64.backward(dout.double().transpose(1, 2))
    lse = oracle.attention_lse(q, k, scale, causal)
    torch.testing.assert_close(lse.double(), lse64.detach(), rtol=1e-6, atol=1e-6)
    out = out64.detach().float().transpose(1, 2).contiguous()
    dq, dk, dv = oracle.attention_backward(dout, q, k, v, out, lse, scale, causal)
    for got, want in ((dq, q64.grad), (dk, k64.grad), (dv, v64.grad)):
        torch.testing.assert_close(got.double(), want, rtol=2e-5, atol=2e-5)


def test_attention_backward_oracle_catches_its_plausible_mistakes():
    """Dropping delta, the scale on dS, or the causal rule each moves a gradient far outside the
    tolerance above: the pin would notice."""
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(1, 2, 6, 8, generator=g) for _ in range(3))
    dout = torch.randn(1, 6, 2, 8, generator=g)
    scale = 0.5
    out = oracle.attention(q, k, v, scale, True)
    lse = oracle.attention_lse(q, k, scale, True)
    dq, dk, dv = oracle.attention_backward(dout, q, k, v, out, lse, scale, True)
    # delta dropped == out replaced by zeros; causal dropped == causal False with the causal lse
    no_delta = oracle.attention_backward(dout, q, k, v, torch.zeros_like(out), lse, scale, True)
    assert (no_delta[0] - dq).abs().max() > 1e-2
    # dv of a hidden key row gets mass only if the causal rule is dropped: key 5 is seen by query 5 alone
    not_causal = oracle.attention_backward(dout, q, k, v, out, lse, scale, False)
    assert (not_causal[2] - dv).abs().max() > 1e-2
    # linearity in dout (dq, dk, dv are linear maps of it for fixed q, k, v, out-consistent delta)
    out2 = oracle.attention_backward(2 * dout, q, k, v, out, lse, scale, True)
    for a2, a1 in zip(out2, (dq, dk, dv)):
        torch.testing.assert_close(a2, 2 * a1, rtol=1e-5, atol=1e-6)
    # sum over keys of dS is zero for every query (softmax rows sum to one), so adding a constant
    # vector c to every key leaves dq unchanged up to rounding: dq = dS K
    shifted = oracle.attention_backward(dout, q, k + 3.0, v, oracle.attention(q, k + 3.0, v, scale, True),
                                        oracle.attention_lse(q, k + 3.0, scale, True), scale, True)
    torch.testing.assert_close(shifted[0], dq, rtol=1e-3, atol=1e-4)
