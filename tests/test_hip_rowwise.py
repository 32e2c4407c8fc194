"""GPU parity of softmax / log_softmax / native_layer_norm: HIP kernels (through the C ABI)
against the CPU oracle and the float64 closed forms, on seeded inputs."""

import numpy as np
import pytest
import torch

import oracle
from oracle import closed_form as cf
from helpers import as64, assert_close64, seeded

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _dev(t):
    return t.to("cuda")


def _ops():
    from torch_mojo_backend.eager_kernels import hip_ops
    return hip_ops


# cols chosen to hit every register-resident configuration, the 16-wave one, the generic
# fallback (unaligned widths, beyond-register widths) and the GPT-2 / benchmark shapes.
SOFTMAX_SHAPES = [(7, 1), (5, 8), (33, 257), (64, 64), (19, 128), (300, 768), (130, 1024),
                  (67, 2048), (35, 4096), (9, 8192), (5, 16384), (3, 32768), (2, 40000),
                  (4, 50257), (3, 70000),
                  # long ragged rows (one 1024-thread workgroup per row, unaligned vectors): each
                  # vector count per lane, tails of 1 .. 7 elements, the widest row it takes
                  (37, 4099), (5, 16389), (6, 30001), (3, 65535), (130, 50257)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", SOFTMAX_SHAPES)
@pytest.mark.parametrize("log", [False, True])
def test_softmax_matches_oracle(shape, dtype, log):
    x = seeded(shape, seed=shape[1], scale=4.0, dtype=dtype)
    got = _ops().softmax(_dev(x), -1, log=log)
    assert got.dtype == dtype and tuple(got.shape) == shape
    want = (cf.log_softmax if log else cf.softmax)(as64(x))
    assert_close64(got, want, what=f"softmax{shape} log={log}")
    # and against the C restatement of the reference CPU kernel
    # the reference kernel sums its denominator sequentially in fp32: cols * 2^-24 a priori
    ref = oracle.softmax_rows(x, log=log)
    seq = shape[1] * 2.0 ** -24
    assert_close64(got, as64(ref), rtol=2e-5 + seq, atol=2e-6 + (seq if log else 0.0),
                   rounded_want=True, what="vs C oracle")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(37, 1024), (9, 50257)])
def test_softmax_half_to_float(dtype, shape):
    x = seeded(shape, seed=3, scale=4.0, dtype=dtype)
    got = _ops().softmax(_dev(x), -1, half_to_float=True)
    assert got.dtype == torch.float32
    assert_close64(got, cf.softmax(as64(x)), what="half_to_float")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("log", [False, True])
def test_softmax_long_rows_at_an_odd_address(dtype, log):
    """Whole vectors per row, but the tensor starts one element past a 16-byte boundary (a slice
    of a larger buffer): the unaligned long-row kernel, with nothing written outside the rows."""
    rows, cols = 6, 8192
    x = seeded((rows, cols), seed=11, scale=4.0, dtype=dtype)
    buf = torch.zeros(rows * cols + 1, dtype=dtype, device="cuda")
    view = buf[1:].view(rows, cols)
    view.copy_(x)
    assert view.data_ptr() % 16 != 0
    got = _ops().softmax(view, -1, log=log)
    want = (cf.log_softmax if log else cf.softmax)(as64(x))
    assert_close64(got, want, what=f"odd address log={log} {dtype}")
    assert float(buf[0]) == 0.0 and torch.equal(view.cpu(), x)


@pytest.mark.parametrize("dim", [0, 1, 2, -1, -2])
def test_softmax_any_dim(dim):
    x = seeded((6, 10, 12), seed=11, scale=2.0)
    got = _ops().softmax(_dev(x), dim)
    assert_close64(got, cf.softmax(as64(x), axis=dim), what=f"dim={dim}")
    assert got.shape == x.shape


def test_softmax_invariants_full_size():
    """Benchmark-size rows: sums to one and shift invariance (size-independent properties)."""
    x = seeded((4096, 4096), seed=5, scale=4.0)
    xd = _dev(x)
    p = _ops().softmax(xd, -1)
    sums = p.double().sum(-1).cpu().numpy()
    assert np.abs(sums - 1.0).max() < 1e-5
    assert (p >= 0).all()
    shifted = _ops().softmax(xd + 3.0, -1)
    assert torch.allclose(p, shifted, rtol=2e-5, atol=1e-7)
    # argmax of probabilities is the argmax of the logits
    assert torch.equal(p.argmax(-1).cpu(), x.argmax(-1))


def test_softmax_extremes():
    x = torch.tensor([[1e4, -1e4, 0.0, 1e4], [-1e30, -1e30, -1e30, -1e30],
                      [float("-inf"), 0.0, 1.0, 2.0], [88.0, 89.0, -88.0, 0.0]])
    got = _ops().softmax(_dev(x), -1)
    assert_close64(got, cf.softmax(as64(x)), what="extremes")
    nan_row = torch.tensor([[1.0, float("nan"), 2.0, 3.0]])
    assert torch.isnan(_ops().softmax(_dev(nan_row), -1)).all()


def test_softmax_rank0_and_offset_storage():
    ops = _ops()
    assert ops.softmax(_dev(torch.tensor(3.0)), -1).item() == 1.0
    assert ops.softmax(_dev(torch.tensor(3.0)), -1, log=True).item() == 0.0
    base = seeded((5 * 64 + 1,), seed=2)
    view = _dev(base)[1:].view(5, 64)  # 4-byte aligned only: must take the generic kernel
    assert_close64(ops.softmax(view, -1), cf.softmax(as64(base[1:].view(5, 64))), what="offset")


LN_SHAPES = [(3, 7), (6, 768), (5, 769), (3, 65), (16, 1024), (33, 2048), (9, 4096), (4, 8192),
             (3, 16384), (2, 40000), (257, 768)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", LN_SHAPES)
def test_layer_norm_matches_oracle(shape, dtype):
    rows, cols = shape
    x = seeded(shape, seed=cols, dtype=dtype)
    g = seeded((cols,), seed=1, scale=0.1, shift=1.0, dtype=dtype)
    b = seeded((cols,), seed=2, scale=0.1, dtype=dtype)
    out, mean, rstd = _ops().layer_norm(_dev(x), [cols], _dev(g), _dev(b), 1e-5)
    assert out.dtype == dtype and mean.dtype == torch.float32 and rstd.dtype == torch.float32
    assert tuple(mean.shape) == (rows, 1) and tuple(rstd.shape) == (rows, 1)
    w_out, w_mean, w_rstd = cf.layer_norm(as64(x), as64(g), as64(b), 1e-5)
    # out = (x-mean)*rstd*g+b: error scales with |x-mean|*rstd*|g|, so allow rtol on that scale
    scale = np.abs(as64(x) - w_mean) * w_rstd * np.abs(as64(g)) + np.abs(as64(b))
    assert_close64(out, w_out, extra_abs=1e-5 * scale, what=f"ln out {shape}")
    assert_close64(mean, w_mean, atol=1e-6, what="ln mean")
    assert_close64(rstd, w_rstd, rtol=1e-5, what="ln rstd")
    r_out, r_mean, r_rstd = oracle.layer_norm_rows(x, g, b, 1e-5)
    seq = cols * 2.0 ** -24  # sequential fp32 sums in the reference kernel
    assert_close64(mean.reshape(-1), as64(r_mean), atol=2e-6 + seq * np.abs(as64(x)).mean(-1),
                   rounded_want=True, what="mean vs C oracle")
    assert_close64(rstd.reshape(-1), as64(r_rstd), rtol=2e-5 + seq, rounded_want=True,
                   what="rstd vs C oracle")


# Row widths on both sides of every geometry switch of the kernel (lanes per row x vectors per
# lane, in 16-byte input vectors: 16x1 .. 1024x16), for 4- and 2-byte inputs, with row counts that
# leave the last workgroup and the last iteration of the persistent walk partly empty.
LN_WIDTHS_VEC = [1, 15, 16, 17, 32, 33, 48, 49, 64, 65, 96, 97, 128, 129, 192, 193, 256, 257, 384,
                 385, 512, 513, 768, 769, 1024, 1025, 2048, 2049, 4096, 4100]


@pytest.mark.parametrize("nvec", LN_WIDTHS_VEC)
@pytest.mark.parametrize("in_dtype,out_dtype", [(torch.float32, torch.float32),
                                                (torch.bfloat16, torch.bfloat16),
                                                (torch.float32, torch.bfloat16),
                                                (torch.float32, torch.float16)])
def test_layer_norm_every_geometry_and_the_widening_input(nvec, in_dtype, out_dtype):
    cols = nvec * (4 if in_dtype == torch.float32 else 8)
    rows = 37 if cols <= 4096 else 5
    x = seeded((rows, cols), seed=nvec, scale=2.0, shift=0.25, dtype=in_dtype)
    g = seeded((cols,), seed=1, scale=0.1, shift=1.0, dtype=out_dtype)
    b = seeded((cols,), seed=2, scale=0.1, dtype=out_dtype)
    out, mean, rstd = _ops().layer_norm(_dev(x), [cols], _dev(g), _dev(b), 1e-5, out_dtype=out_dtype)
    assert out.dtype == out_dtype and mean.dtype == torch.float32 and tuple(mean.shape) == (rows, 1)
    w_out, w_mean, w_rstd = cf.layer_norm(as64(x), as64(g), as64(b), 1e-5)
    scale = np.abs(as64(x) - w_mean) * w_rstd * np.abs(as64(g)) + np.abs(as64(b))
    assert_close64(out, w_out, extra_abs=1e-5 * scale, what=f"ln out {rows}x{cols}")
    assert_close64(mean, w_mean, atol=2e-6, what="ln mean")
    assert_close64(rstd, w_rstd, rtol=1e-5, what="ln rstd")


def test_layer_norm_widening_input_rejects_other_combinations():
    x = _dev(seeded((4, 64), dtype=torch.bfloat16))
    with pytest.raises(TypeError, match="cannot be normalised"):
        _ops().layer_norm(x, [64], None, None, 1e-5, out_dtype=torch.float32)
    xf = _dev(seeded((4, 64)))
    w16 = _dev(seeded((64,), dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="weight must be"):
        _ops().layer_norm(xf, [64], w16, None, 1e-5)                       # fp32 out wants fp32 weight
    out, _, _ = _ops().layer_norm(xf, [64], w16, None, 1e-5, out_dtype=torch.bfloat16)
    assert out.dtype == torch.bfloat16


def test_layer_norm_full_size_rows_walk_whole_tensor():
    """The persistent walk at the benchmark shapes: every row is written exactly once and matches
    a float64 reference on sampled rows (first, last, and the rows around each workgroup's stride)."""
    for rows, cols, dtype in ((32768, 768, torch.bfloat16), (16384, 4096, torch.float32),
                              (32768, 768, torch.float32)):
        g_ = torch.Generator(device="cuda").manual_seed(rows + cols)
        x = (torch.randn(rows, cols, generator=g_, device="cuda") * 1.5 + 0.3).to(dtype)
        w = (1 + 0.1 * torch.randn(cols, generator=g_, device="cuda")).to(dtype)
        b = (0.1 * torch.randn(cols, generator=g_, device="cuda")).to(dtype)
        out, mean, rstd = _ops().layer_norm(x, [cols], w, b, 1e-5)
        assert not torch.isnan(out).any()
        pick = torch.tensor([0, 1, 7, 8, 1023, 1024, 4095, 4096, 8191, 8192, rows // 2, rows - 2, rows - 1])
        xs = x[pick].double().cpu()
        want = torch.nn.functional.layer_norm(xs, [cols], w.double().cpu(), b.double().cpu(), 1e-5)
        tol = 2e-2 if dtype == torch.bfloat16 else 2e-5
        torch.testing.assert_close(out[pick].double().cpu(), want, rtol=tol, atol=tol)
        torch.testing.assert_close(mean[pick, 0].double().cpu(), xs.mean(-1), rtol=1e-5, atol=2e-6)
        # every row normalised: per-row mean of (out - b) / w is ~0
        z = ((out.float() - b.float()) / w.float()).mean(-1).abs().max().item()
        assert z < (3e-2 if dtype == torch.bfloat16 else 1e-4)


@pytest.mark.parametrize("has_weight,has_bias", [(False, False), (True, False), (False, True)])
@pytest.mark.parametrize("shape,normalized,eps", [((3, 7), (7,), 1e-5), ((2, 3, 4), (3, 4), 0.5)])
def test_layer_norm_optional_affine(shape, normalized, eps, has_weight, has_bias):
    x = seeded(shape, seed=20260720 % 1000)
    w = seeded(normalized, seed=4) if has_weight else None
    b = seeded(normalized, seed=5) if has_bias else None
    out, mean, rstd = _ops().layer_norm(_dev(x), list(normalized), None if w is None else _dev(w),
                                        None if b is None else _dev(b), eps)
    want = torch.native_layer_norm(x, normalized, w, b, eps)
    for got, ref, tol in zip((out, mean, rstd), want, (1e-5, 1e-5, 1e-4)):
        torch.testing.assert_close(got.cpu(), ref, atol=tol, rtol=tol)
    k = len(normalized)
    assert tuple(mean.shape) == tuple(shape[:-k]) + (1,) * k


@pytest.mark.parametrize("cols", [768, 769])
@pytest.mark.parametrize("value", [float("nan"), float("inf"), float("-inf")])
def test_layer_norm_nonfinite_rows(cols, value):
    x = torch.full((2, cols), value)
    out, mean, rstd = _ops().layer_norm(_dev(x), [cols], None, None, 1e-5)
    assert torch.isnan(out).all() and torch.isnan(mean).all() and torch.isnan(rstd).all()


def test_layer_norm_without_stats_and_invariants():
    x = seeded((8192, 768), seed=9, scale=3.0, shift=0.5)
    out, mean, rstd = _ops().layer_norm(_dev(x), [768], None, None, 1e-5, need_stats=False)
    assert mean is None and rstd is None
    o = out.double()
    assert o.mean(-1).abs().max().item() < 1e-5          # gamma=1, beta=0 => zero mean
    assert (o.var(-1, unbiased=False) - 1).abs().max().item() < 1e-3  # ... and unit variance


def test_row_kernels_are_deterministic():
    """Queue three launches before syncing; outputs must be bit-identical."""
    x = _dev(seeded((2048, 1024), seed=1, scale=4.0))
    outs = [_ops().softmax(x, -1) for _ in range(3)]
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])


# ---------------------------------------------------------------- attention softmax (scale, causal)
# widths pick every kernel family: one wave per row (64, 128, 1024), several waves per row
# (4096 fp32), the generic kernel (77: not a whole number of 16-byte vectors)
SCALED_SHAPES = [(2, 3, 64, 64), (1, 2, 128, 128), (3, 1000, 1000), (2, 1024, 1024), (1, 77, 77),
                 (1, 300, 4096)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", SCALED_SHAPES)
@pytest.mark.parametrize("causal", [False, True])
def test_softmax_scaled_matches_oracle(shape, dtype, causal):
    q_len = shape[-2]  # (300, 4096) is rectangular: keys beyond the query index are masked too
    x = seeded(shape, seed=31, scale=4.0, dtype=dtype)
    scale = 0.125
    got = _ops().softmax_scaled(_dev(x), scale, causal_q_len=q_len if causal else 0)
    assert got.dtype == dtype and got.shape == x.shape
    want = cf.softmax_scaled_causal(as64(x), scale, causal)
    cols = shape[-1]
    assert_close64(got, want, rtol=1e-5, atol=1e-6 + cols * 2.0 ** -24 * 1e-2, what="vs closed form")
    ref = oracle.softmax_scaled(x, scale, causal_q_len=q_len if causal else 0)
    assert_close64(got, as64(ref), rtol=1e-5, atol=1e-6 + cols * 2.0 ** -24, rounded_want=True,
                   what="vs C oracle")
    if causal:
        upper = torch.ones(shape[-2], shape[-1], dtype=torch.bool).triu(1)
        assert bool((got.cpu()[..., upper] == 0).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_softmax_scaled_rounding_reproduces_the_three_op_pipeline(dtype):
    """round_scaled: bit-identical to mul -> masked_fill(-inf) -> softmax run one after another."""
    x = _dev(seeded((4, 6, 256, 256), seed=32, scale=3.0, dtype=dtype))
    mask = _dev(torch.tril(torch.ones(256, 256)) == 0)
    scale = 1.0 / 8.0 + 1.0 / 64.0  # not a power of two: the product really rounds
    unfused = _ops().softmax((x * scale).masked_fill(mask, float("-inf")), -1)
    fused = _ops().softmax_scaled(x, scale, causal_q_len=256, round_scaled=True)
    assert torch.equal(fused, unfused)


def test_softmax_scaled_full_size_invariants():
    """Benchmark attention shape [32*12, 1024, 1024] bf16: rows sum to one, zeros above the
    diagonal, first row is exactly [1, 0, ...]."""
    g = torch.Generator(device="cuda").manual_seed(5)
    x = (torch.randn(96, 1024, 1024, generator=g, device="cuda") * 4).bfloat16()
    y = _ops().softmax_scaled(x, 0.125, causal_q_len=1024)
    sums = y.float().sum(-1)
    assert (sums - 1).abs().max().item() <= 2e-2
    assert bool((y[:, 0, 0] == 1).all()) and bool((y[:, 0, 1:] == 0).all())
    assert bool((y.triu(1) == 0).all())
    assert torch.equal(y, _ops().softmax_scaled(x, 0.125, causal_q_len=1024))


def test_softmax_scaled_rejects_bad_arguments():
    x = _dev(seeded((2, 8, 8), dtype=torch.float32))
    with pytest.raises(ValueError):
        _ops().softmax_scaled(x, 1.0, causal_q_len=4)      # q_len must be the query dimension
    with pytest.raises(TypeError, match="no CPU path"):
        _ops().softmax_scaled(x.cpu(), 1.0)
