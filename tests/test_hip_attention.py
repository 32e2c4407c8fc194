"""GPU parity of the fused attention forward (scores never reach memory)."""

import numpy as np
import pytest
import torch

import oracle
from oracle import closed_form as cf
from helpers import as64, seeded

pytestmark = pytest.mark.gpu


def _ops():
    from torch_mojo_backend.eager_kernels import hip_ops
    return hip_ops


def _qkv(b, h, t, s, dtype, seed=0):
    return (seeded((b, h, t, 64), seed=seed, dtype=dtype), seeded((b, h, s, 64), seed=seed + 1, dtype=dtype),
            seeded((b, h, s, 64), seed=seed + 2, dtype=dtype))


# query/key counts around the 128-query workgroup, the 32-query wave and the 64-key block
SHAPES = [(1, 1, 1, 1), (2, 3, 33, 33), (1, 2, 64, 64), (2, 2, 65, 65), (1, 3, 128, 128),
          (1, 2, 129, 129), (2, 4, 200, 200), (1, 2, 77, 150), (1, 2, 150, 77), (1, 12, 512, 512)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("btsh", SHAPES)
@pytest.mark.parametrize("causal", [False, True])
def test_attention_matches_closed_form_and_oracle(btsh, dtype, causal):
    b, h, t, s = btsh
    q, k, v = _qkv(b, h, t, s, dtype, seed=t + s)
    scale = 0.125
    got = _ops().attention(q.cuda(), k.cuda(), v.cuda(), scale, causal)
    assert got.shape == (b, t, h, 64) and got.dtype == dtype and got.is_contiguous()
    want = cf.attention(as64(q), as64(k), as64(v), scale, causal)
    # probabilities are stored with the storage type's 8 (bf16) / 11 (fp16) bit significand and
    # the output once more: |error| <= 2 ulp of the largest |v| that is averaged (about 4.5)
    tol = {torch.bfloat16: 3e-2, torch.float16: 4e-3}[dtype]
    err = np.abs(as64(got) - want)
    assert err.max() <= tol, f"max err {err.max():.3e}"
    assert err.mean() <= tol / 8
    ref = oracle.attention(q, k, v, scale, causal)
    assert np.abs(as64(got) - as64(ref)).max() <= 2 * tol


@pytest.mark.parametrize("causal", [False, True])
def test_attention_special_cases(causal):
    # identical keys -> uniform weights -> running mean of the values (causal) or their mean
    v = seeded((1, 2, 96, 64), seed=3, dtype=torch.float16)
    k = torch.ones(1, 2, 96, 64, dtype=torch.float16)
    q = seeded((1, 2, 96, 64), seed=4, dtype=torch.float16) * 0.01
    got = as64(_ops().attention(q.cuda(), k.cuda(), v.cuda(), 1.0, causal))
    v64 = as64(v)
    if causal:
        want = np.cumsum(v64, axis=2) / np.arange(1, 97)[None, None, :, None]
    else:
        want = np.broadcast_to(v64.mean(axis=2, keepdims=True), v64.shape)
    np.testing.assert_allclose(got, want.transpose(0, 2, 1, 3), atol=3e-3)
    # huge scores must not overflow: one dominant key per query
    q2 = torch.zeros(1, 1, 64, 64, dtype=torch.bfloat16)
    k2 = torch.zeros(1, 1, 64, 64, dtype=torch.bfloat16)
    q2[..., 0] = 200.0
    k2[0, 0, 0, 0] = 200.0                  # key 0 scores 40000 * scale, the rest 0
    v2 = seeded((1, 1, 64, 64), seed=5, dtype=torch.bfloat16)
    got2 = _ops().attention(q2.cuda(), k2.cuda(), v2.cuda(), 1.0, causal).cpu()
    assert torch.isfinite(got2).all()
    assert torch.equal(got2[0, :, 0], v2[0, 0, 0].expand(64, 64))


def test_attention_reads_a_packed_projection_in_place():
    """q, k, v as strided slices of one [B, T, 3*H*64] tensor, exactly as a decoder block holds
    them: no copies, same numbers as the contiguous call."""
    b, t, h = 2, 256, 12
    qkv = seeded((b, t, 3 * h * 64), seed=9, dtype=torch.bfloat16).cuda()
    q, k, v = (x.view(b, t, h, 64).transpose(1, 2) for x in qkv.split(h * 64, dim=2))
    assert not q.is_contiguous() and _ops().attention_supported(q, k, v)
    got = _ops().attention(q, k, v, 0.125, True)
    same = _ops().attention(q.contiguous(), k.contiguous(), v.contiguous(), 0.125, True)
    assert torch.equal(got, same)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.float().cpu(), k.float().cpu(), v.float().cpu(), is_causal=True, scale=0.125)
    assert (got.float().cpu() - want.transpose(1, 2)).abs().max().item() <= 3e-2


def test_attention_benchmark_shape_and_determinism():
    """GPT-2 small at B=32, T=1024: [32, 12, 1024, 64] bf16, causal. Checked on sampled
    (batch, head) pairs against float64 and for bit-identical repeats."""
    g = torch.Generator(device="cuda").manual_seed(0)
    qkv = torch.randn(32, 1024, 2304, generator=g, device="cuda").bfloat16()
    q, k, v = (x.view(32, 1024, 12, 64).transpose(1, 2) for x in qkv.split(768, dim=2))
    got = _ops().attention(q, k, v, 0.125, True, round_like_unfused=True)
    assert torch.equal(got, _ops().attention(q, k, v, 0.125, True, round_like_unfused=True))
    for (bi, hi) in ((0, 0), (17, 5), (31, 11)):
        want = cf.attention(as64(q[bi:bi + 1, hi:hi + 1]), as64(k[bi:bi + 1, hi:hi + 1]),
                            as64(v[bi:bi + 1, hi:hi + 1]), 0.125, True)
        err = np.abs(as64(got[bi:bi + 1, :, hi:hi + 1]) - want)
        assert err.max() <= 3e-2 and err.mean() <= 3e-3


def test_attention_rejects_what_it_cannot_take():
    ops = _ops()
    q, k, v = (x.cuda() for x in _qkv(1, 1, 8, 8, torch.bfloat16))
    assert not ops.attention_supported(q.float(), k.float(), v.float())
    assert not ops.attention_supported(q[..., :32], k[..., :32], v[..., :32])
    assert not ops.attention_supported(q.cpu(), k.cpu(), v.cpu())
    with pytest.raises(ValueError):
        ops.attention(q[..., :32], k[..., :32], v[..., :32], 1.0, True)


def test_registry_entry_for_scaled_dot_product_attention():
    """aten.scaled_dot_product_attention: HIP kernel when it can take the call, PyTorch-ROCm's
    op otherwise; same shape and layout contract ([batch, heads, tokens, head_dim])."""
    from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO
    fn = MAPPING_TORCH_ATEN_TO_MOJO[torch.ops.aten.scaled_dot_product_attention]
    q, k, v = (x.cuda() for x in _qkv(2, 4, 100, 100, torch.bfloat16, seed=5))
    got = fn(q, k, v, is_causal=True)
    assert got.shape == (2, 4, 100, 64)
    want = cf.attention(as64(q), as64(k), as64(v), 0.125, True).transpose(0, 2, 1, 3)
    assert np.abs(as64(got) - want).max() <= 3e-2
    # float32 and an explicit mask are not the fused kernel's: GEMM + softmax + GEMM answers
    mask = torch.ones(100, 100, dtype=torch.bool, device="cuda").tril()
    via_mask = fn(q, k, v, attn_mask=mask)
    assert np.abs(as64(via_mask) - want).max() <= 3e-2
    f32 = fn(q.float(), k.float(), v.float(), is_causal=True)
    assert f32.dtype == torch.float32 and np.abs(as64(f32) - want).max() <= 1e-4


def test_eager_device_scaled_dot_product_attention():
    from torch_mojo_backend import register_mojo_devices
    from torch_mojo_backend.eager_kernels import aten_fast
    register_mojo_devices()
    from torch_mojo_backend.mojo_device.torch_mojo_tensor import TorchMojoTensor
    q, k, v = (x.cuda() for x in _qkv(1, 2, 70, 70, torch.float16, seed=8))
    wrap = lambda t: aten_fast._wrap(t)  # noqa: E731
    out = aten_fast.fast_aten_scaled_dot_product_attention(wrap(q), wrap(k), wrap(v), is_causal=True)
    assert isinstance(out, TorchMojoTensor) and tuple(out._shape) == (1, 2, 70, 64)
    want = cf.attention(as64(q), as64(k), as64(v), 0.125, True).transpose(0, 2, 1, 3)
    assert np.abs(as64(out._holder) - want).max() <= 4e-3
    # what it cannot take is handed back
    assert aten_fast.fast_aten_scaled_dot_product_attention(
        wrap(q), wrap(k), wrap(v), dropout_p=0.1) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_scaled_dot_product_attention(
        wrap(q), wrap(k), wrap(v), enable_gqa=True) is aten_fast.NOT_HANDLED
    # float32 goes through GEMM + softmax + GEMM
    f32 = aten_fast.fast_aten_scaled_dot_product_attention(
        wrap(q.float()), wrap(k.float()), wrap(v.float()), is_causal=True)
    assert isinstance(f32, TorchMojoTensor) and f32._dtype == torch.float32
    want32 = cf.attention(as64(q), as64(k), as64(v), 0.125, True).transpose(0, 2, 1, 3)
    assert np.abs(as64(f32._holder) - want32).max() <= 1e-4


# ---- composed attention: GEMM + softmax + GEMM for what the fused kernel does not take ----------
def _sdpa64(q, k, v, scale, causal, mask):
    """float64 closed form with an optional boolean / additive mask."""
    s = np.einsum("...td,...sd->...ts", as64(q), as64(k)) * scale
    t, n = s.shape[-2], s.shape[-1]
    if causal:
        s = np.where(np.tril(np.ones((t, n), dtype=bool)), s, -np.inf)
    if mask is not None:
        m = mask.numpy()
        s = np.where(m, s, -np.inf) if m.dtype == np.bool_ else s + m.astype(np.float64)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("...ts,...sd->...td", p, as64(v))


@pytest.mark.parametrize("case", [
    # (shape of q, keys, head_dim_v, dtype, causal, mask kind)
    ((2, 3, 17, 32), 17, 32, torch.float32, True, None),
    ((2, 3, 17, 32), 29, 48, torch.float32, False, "bool"),
    ((1, 4, 40, 128), 40, 128, torch.bfloat16, True, None),
    ((2, 12, 1, 64), 37, 64, torch.bfloat16, False, None),      # a decode step
    ((2, 2, 9, 64), 21, 64, torch.float16, False, "float"),
    ((3, 5, 80), 80, 80, torch.float32, False, None),           # no head dimension
])
def test_attention_composed_matches_closed_form(case):
    qshape, keys, dv, dtype, causal, kind = case
    q = seeded(qshape, seed=1, dtype=dtype)
    k = seeded(qshape[:-2] + (keys, qshape[-1]), seed=2, dtype=dtype)
    v = seeded(qshape[:-2] + (keys, dv), seed=3, dtype=dtype)
    mask = None
    if kind == "bool":
        g = torch.Generator().manual_seed(5)
        mask = torch.rand(qshape[0], 1, qshape[-2], keys, generator=g) > 0.3
        mask[..., 0] = True  # every query keeps at least one key
    elif kind == "float":
        mask = seeded((qshape[-2], keys), seed=6, dtype=dtype)
    scale = 1.0 / np.sqrt(qshape[-1])
    got = _ops().attention_composed(q.cuda(), k.cuda(), v.cuda(), scale, causal,
                                    None if mask is None else mask.cuda())
    assert got.shape == qshape[:-1] + (dv,) and got.dtype == dtype
    want = _sdpa64(q, k, v, scale, causal, mask)
    tol = {torch.float32: 2e-5, torch.bfloat16: 4e-2, torch.float16: 5e-3}[dtype]
    assert np.abs(as64(got) - want).max() <= tol
    # and PyTorch's CPU op on the same inputs (fp32 only: its 16-bit CPU path rounds differently)
    if dtype == torch.float32 and q.dim() == 4:
        ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, is_causal=causal)
        torch.testing.assert_close(got.cpu(), ref, rtol=1e-4, atol=1e-5)


def test_sdpa_surfaces_use_the_composed_path_for_fp32_and_masks():
    from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO, register_mojo_devices
    register_mojo_devices()
    q = seeded((2, 4, 12, 32), seed=1)
    k = seeded((2, 4, 20, 32), seed=2)
    v = seeded((2, 4, 20, 32), seed=3)
    mask = torch.ones(12, 20, dtype=torch.bool).tril(8)
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    fn = MAPPING_TORCH_ATEN_TO_MOJO[torch.ops.aten.scaled_dot_product_attention]
    torch.testing.assert_close(fn(q.cuda(), k.cuda(), v.cuda(), mask.cuda()).cpu(), want, rtol=1e-4, atol=1e-5)
    got = torch.nn.functional.scaled_dot_product_attention(q.to("mojo"), k.to("mojo"), v.to("mojo"),
                                                           attn_mask=mask.to("mojo"))
    assert got.device.type == "mojo"
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-5)


# ---- decode kernel: a few queries per head, K and V read once ------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", [
    # (batch, heads, queries, keys, head_dim, causal, mask)
    (2, 3, 1, 1, 64, False, False), (4, 12, 1, 37, 64, False, True), (2, 2, 1, 208, 64, False, False),
    (1, 2, 5, 64, 64, True, False), (2, 4, 16, 100, 64, False, True), (3, 2, 1, 333, 128, False, True),
    (1, 3, 7, 7, 128, True, False), (2, 2, 2, 1000, 64, False, False),
])
def test_attention_decode_matches_closed_form(case, dtype):
    b, h, t, s, d, causal, with_mask = case
    q = seeded((b, h, t, d), seed=1, dtype=dtype)
    k = seeded((b, h, s, d), seed=2, dtype=dtype)
    v = seeded((b, h, s, d), seed=3, dtype=dtype)
    mask = None
    if with_mask:
        mask = torch.rand(b, 1, t, s, generator=torch.Generator().manual_seed(9)) > 0.3
        mask[..., 0] = True
    scale = 1.0 / np.sqrt(d)
    assert _ops().attention_decode_supported(q.cuda(), k.cuda(), v.cuda(), None if mask is None else mask.cuda())
    got = _ops().attention_decode(q.cuda(), k.cuda(), v.cuda(), scale, causal,
                                  None if mask is None else mask.cuda())
    assert got.shape == (b, h, t, d) and got.dtype == dtype and got.is_contiguous()
    want = _sdpa64(q, k, v, scale, causal, mask)
    tol = {torch.bfloat16: 2e-2, torch.float16: 3e-3}[dtype]
    assert np.abs(as64(got) - want).max() <= tol


def test_attention_decode_strided_views_masked_rows_and_rejections():
    ops = _ops()
    # q/k/v as the thirds of a packed projection (strided heads), keys as a slice of a longer cache
    b, h, t, s, d = 2, 4, 1, 50, 64
    qkv = seeded((b, t, 3 * h * d), seed=4, dtype=torch.bfloat16).cuda()
    q = qkv[..., :h * d].view(b, t, h, d).transpose(1, 2)
    cache = seeded((2, b, h, 128, d), seed=5, dtype=torch.bfloat16).cuda()
    k, v = cache[0, :, :, :s], cache[1, :, :, :s]
    got = ops.attention_decode(q, k, v, 0.125, False, None)
    want = _sdpa64(q.cpu(), k.cpu(), v.cpu(), 0.125, False, None)
    assert np.abs(as64(got) - want).max() <= 2e-2
    # a query whose keys are all masked out yields NaN, like ATen
    mask = torch.ones(b, 1, t, s, dtype=torch.bool)
    mask[1] = False
    out = ops.attention_decode(q, k, v, 0.125, False, mask.cuda()).float().cpu()
    assert torch.isnan(out[1]).all() and not torch.isnan(out[0]).any()
    # what it does not take
    assert not ops.attention_decode_supported(q.float(), k.float(), v.float(), None)
    assert not ops.attention_decode_supported(q, k, v, torch.zeros(t, s, device="cuda"))  # additive
    big_q = seeded((b, h, 17, d), seed=6, dtype=torch.bfloat16).cuda()
    assert not ops.attention_decode_supported(big_q, k, v, None)


def test_sdpa_surfaces_route_decode_shapes_to_the_decode_kernel(monkeypatch):
    from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO
    from torch_mojo_backend.eager_kernels import hip_ops
    calls = []
    real = hip_ops.attention_decode
    monkeypatch.setattr(hip_ops, "attention_decode", lambda *a, **kw: calls.append(1) or real(*a, **kw))
    q = seeded((2, 4, 1, 64), seed=1, dtype=torch.bfloat16).cuda()
    k = seeded((2, 4, 30, 64), seed=2, dtype=torch.bfloat16).cuda()
    v = seeded((2, 4, 30, 64), seed=3, dtype=torch.bfloat16).cuda()
    mask = torch.ones(2, 1, 1, 30, dtype=torch.bool, device="cuda")
    fn = MAPPING_TORCH_ATEN_TO_MOJO[torch.ops.aten.scaled_dot_product_attention]
    got = fn(q, k, v, mask)
    assert calls and got.shape == (2, 4, 1, 64)
    want = _sdpa64(q.cpu(), k.cpu(), v.cpu(), 0.125, False, mask.cpu())
    assert np.abs(as64(got) - want).max() <= 2e-2


def test_unmasked_decode_step_takes_the_decode_kernel(monkeypatch):
    """is_causal=False, no mask, one query per head: the graph mapping must
    pick the memory-bound decode kernel, not the 128-query MFMA kernel (which also accepts the
    shapes)."""
    from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO
    from torch_mojo_backend.eager_kernels import hip_ops
    decode_calls, fused_calls = [], []
    real_decode, real_fused = hip_ops.attention_decode, hip_ops.attention
    monkeypatch.setattr(hip_ops, "attention_decode",
                        lambda *a, **kw: decode_calls.append(1) or real_decode(*a, **kw))
    monkeypatch.setattr(hip_ops, "attention", lambda *a, **kw: fused_calls.append(1) or real_fused(*a, **kw))
    q = seeded((3, 12, 1, 64), seed=4, dtype=torch.bfloat16).cuda()
    k = seeded((3, 12, 208, 64), seed=5, dtype=torch.bfloat16).cuda()
    v = seeded((3, 12, 208, 64), seed=6, dtype=torch.bfloat16).cuda()
    assert hip_ops.attention_supported(q, k, v)                 # the MFMA kernel would take it too
    want = _sdpa64(q.cpu(), k.cpu(), v.cpu(), 0.125, False, None)
    got = MAPPING_TORCH_ATEN_TO_MOJO[torch.ops.aten.scaled_dot_product_attention](q, k, v)
    assert len(decode_calls) == 1 and not fused_calls
    assert np.abs(as64(got) - want).max() <= 2e-2
    # 17 queries: past the decode kernel's limit, the MFMA kernel takes over
    q17 = seeded((3, 12, 17, 64), seed=7, dtype=torch.bfloat16).cuda()
    MAPPING_TORCH_ATEN_TO_MOJO[torch.ops.aten.scaled_dot_product_attention](q17, k, v)
    assert len(fused_calls) == 1
