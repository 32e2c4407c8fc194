"""GPU parity of the fused attention backward (dq, dk, dv without the probabilities in memory) and
of the log-sum-exp the forward kernel hands it."""

import numpy as np
import pytest
import torch

import oracle
from helpers import as64, seeded

pytestmark = pytest.mark.gpu


def _ops():
    from torch_mojo_backend.eager_kernels import hip_ops
    return hip_ops


def _inputs(b, h, t, s, dtype, seed):
    q, k, v = (seeded((b, h, n, 64), seed=seed + i, dtype=dtype) for i, n in enumerate((t, s, s)))
    dout = seeded((b, t, h, 64), seed=seed + 3, dtype=dtype)
    return q, k, v, dout


def _float64_reference(q, k, v, dout, scale, causal):
    """float64 autograd of softmax(scale q k^T + mask) v on the stored operands."""
    q64, k64, v64 = (x.double().requires_grad_(True) for x in (q, k, v))
    s = (q64 @ k64.transpose(-1, -2)) * scale
    if causal:
        t, n = s.shape[-2:]
        s = s.masked_fill(torch.ones(t, n, dtype=torch.bool).triu(1), float("-inf"))
    out = torch.softmax(s, -1) @ v64
    out.backward(dout.double().transpose(1, 2))
    return out.detach(), torch.logsumexp(s, -1).detach(), q64.grad, k64.grad, v64.grad


def _run(q, k, v, dout, scale, causal):
    ops = _ops()
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    out, lse = ops.attention(qd, kd, vd, scale, causal, return_lse=True)
    grads = ops.attention_backward(dout.cuda().transpose(1, 2), qd, kd, vd, out.transpose(1, 2), lse,
                                   scale, causal)
    return out, lse, grads


# token counts around the 128-row workgroup, the 32-row wave and the 64-row streamed block;
# unequal query / key counts both ways
SHAPES = [(1, 1, 1, 1), (2, 3, 33, 33), (1, 2, 64, 64), (2, 2, 65, 65), (1, 3, 128, 128),
          (1, 2, 129, 129), (2, 4, 200, 200), (1, 2, 77, 150), (1, 2, 150, 77), (1, 2, 300, 40),
          (1, 12, 512, 512)]
# error bound of a gradient relative to its largest entry: P and dS enter their products with the
# storage type's 8 (bf16) / 11 (fp16) bit significand
TOL = {torch.bfloat16: 2e-2, torch.float16: 3e-3}


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("btsh", SHAPES)
@pytest.mark.parametrize("causal", [False, True])
def test_attention_backward_matches_float64_autograd_and_oracle(btsh, dtype, causal):
    b, h, t, s = btsh
    q, k, v, dout = _inputs(b, h, t, s, dtype, seed=3 * t + s)
    scale = 0.125
    out, lse, (dq, dk, dv) = _run(q, k, v, dout, scale, causal)
    _, lse64, *want = _float64_reference(q, k, v, dout, scale, causal)
    assert lse.shape == (b, h, t) and lse.dtype == torch.float32
    np.testing.assert_allclose(as64(lse), lse64.numpy(), rtol=0, atol=2e-5 * (1 + np.abs(lse64.numpy()).max()))
    np.testing.assert_allclose(as64(lse), as64(oracle.attention_lse(q, k, scale, causal)), rtol=0, atol=1e-4)
    ref = oracle.attention_backward(dout, q, k, v, out.cpu(), lse.cpu(), scale, causal)
    floor = 1e-2 * max(w.abs().max().item() for w in want)  # a gradient that is zero by construction
    for name, got, w64, orc in zip("qkv", (dq, dk, dv), want, ref):
        assert got.dtype == dtype and got.shape == w64.shape, name
        big = max(w64.abs().max().item(), floor)
        err = np.abs(as64(got) - w64.numpy())
        assert err.max() <= TOL[dtype] * big, f"d{name}: max err {err.max() / big:.3e} of the largest entry"
        assert err.mean() <= TOL[dtype] * big / 16, f"d{name}: mean err {err.mean() / big:.3e}"
        assert np.abs(as64(got) - as64(orc)).max() <= TOL[dtype] * big, f"d{name} vs oracle"


def test_attention_backward_special_cases():
    # one key: p == 1, dS == 0 up to the summation order of dout . v against dout . out:
    # dq = dk = 0 and dv = sum of the queries' dout
    q, k, v, dout = _inputs(1, 2, 40, 1, torch.float16, seed=9)
    _, _, (dq, dk, dv) = _run(q, k, v, dout, 0.3, False)
    assert dq.abs().max().item() <= 1e-4 and dk.abs().max().item() <= 1e-3
    np.testing.assert_allclose(as64(dv)[:, :, 0], as64(dout).sum(axis=1), rtol=2e-3, atol=2e-3)
    # identical keys and causal: query t spreads dout[t] / (t + 1) over keys 0..t
    v = seeded((1, 1, 96, 64), seed=2, dtype=torch.float16)
    k = torch.ones(1, 1, 96, 64, dtype=torch.float16)
    q = seeded((1, 1, 96, 64), seed=4, dtype=torch.float16) * 0.01
    dout = seeded((1, 96, 1, 64), seed=5, dtype=torch.float16)
    _, _, (_, _, dv) = _run(q, k, v, dout, 1.0, True)
    w = as64(dout)[0, :, 0] / np.arange(1, 97)[:, None]
    want = np.cumsum(w[::-1], axis=0)[::-1]
    np.testing.assert_allclose(as64(dv)[0, 0], want, rtol=0, atol=4e-3 * np.abs(want).max())


def test_attention_backward_reads_packed_projections_and_packs_its_gradients():
    """q, k, v as slices of one [batch, tokens, 3 * heads * 64] projection, out and dout as
    transposed views of [batch, tokens, heads, 64]: nothing is copied, and the three gradients come
    back as slices of one packed buffer in the projection's own layout."""
    b, h, t = 2, 3, 130
    qkv = seeded((b, t, 3 * h * 64), seed=11, dtype=torch.bfloat16)
    dout = seeded((b, t, h, 64), seed=12, dtype=torch.bfloat16)
    qkv_d = qkv.cuda()
    qd, kd, vd = (x.view(b, t, h, 64).transpose(1, 2) for x in qkv_d.split(h * 64, dim=2))
    ops = _ops()
    out, lse = ops.attention(qd, kd, vd, 0.125, True, return_lse=True)
    dq, dk, dv = ops.attention_backward(dout.cuda().transpose(1, 2), qd, kd, vd, out.transpose(1, 2),
                                        lse, 0.125, True, packed=True)
    assert dq.data_ptr() + h * 64 * 2 == dk.data_ptr() and dk.data_ptr() + h * 64 * 2 == dv.data_ptr()
    packed = torch.cat([g.transpose(1, 2).reshape(b, t, h * 64) for g in (dq, dk, dv)], dim=2)
    q, k, v = (x.view(b, t, h, 64).transpose(1, 2).contiguous() for x in qkv.split(h * 64, dim=2))
    _, lse2, grads2 = _run(q, k, v, dout, 0.125, True)
    want = torch.cat([g.transpose(1, 2).reshape(b, t, h * 64) for g in grads2], dim=2)
    assert torch.equal(packed, want) and torch.equal(lse, lse2)


def test_attention_backward_is_deterministic_at_the_benchmark_shape():
    """32 x 12 heads x 1024 tokens, causal (one GPT-2 block of the largest benchmark config):
    no atomics, so two calls agree to the bit; the gradients of the first and the last batch entry
    match float32 autograd of the unfused chain (on the host: autograd over HIP tensors is not
    available in a process that has registered the eager device)."""
    b, h, t = 32, 12, 1024
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn(b, h, t, 64, device="cuda", generator=g).bfloat16() for _ in range(3))
    dout = torch.randn(b, t, h, 64, device="cuda", generator=g).bfloat16()
    ops = _ops()
    out, lse = ops.attention(q, k, v, 0.125, True, return_lse=True)
    first = ops.attention_backward(dout.transpose(1, 2), q, k, v, out.transpose(1, 2), lse, 0.125, True)
    again = ops.attention_backward(dout.transpose(1, 2), q, k, v, out.transpose(1, 2), lse, 0.125, True)
    for a1, a2 in zip(first, again):
        assert torch.equal(a1, a2)
    # the reference chain one batch entry at a time: [12, 1024, 1024] float32 scores
    for bi in (0, b - 1):
        q32, k32, v32 = (x[bi].float().cpu().requires_grad_(True) for x in (q, k, v))
        s = (q32 @ k32.transpose(-1, -2)) * 0.125
        s = s.masked_fill(torch.ones(t, t, dtype=torch.bool).triu(1), float("-inf"))
        (torch.softmax(s, -1) @ v32).backward(dout[bi].float().cpu().transpose(0, 1))
        for name, got, want in zip("qkv", first, (q32.grad, k32.grad, v32.grad)):
            big = want.abs().max().item()
            err = (got[bi].float().cpu() - want).abs()
            assert err.max().item() <= 2e-2 * big, (name, err.max().item() / big)
            assert err.mean().item() <= 2e-2 * big / 16, name


def test_attention_backward_rejects_what_it_cannot_take():
    ops = _ops()
    q, k, v, dout = (x.cuda() for x in _inputs(1, 2, 16, 16, torch.bfloat16, seed=1))
    out, lse = ops.attention(q, k, v, 0.125, True, return_lse=True)
    do, o = dout.transpose(1, 2), out.transpose(1, 2)
    with pytest.raises(ValueError):
        ops.attention_backward(do, q, k, v, o, lse, -1.0, True)
    with pytest.raises(ValueError):
        ops.attention_backward(do, q, k, v, o, lse.double(), 0.125, True)
    with pytest.raises(ValueError):
        ops.attention_backward(do.float(), q, k, v, o, lse, 0.125, True)
    with pytest.raises(ValueError):
        ops.attention_backward(do[:, :, :8], q, k, v, o, lse, 0.125, True)
    with pytest.raises(TypeError):
        ops.attention_backward(do.cpu(), q, k, v, o, lse, 0.125, True)


def test_registry_entries_for_the_flash_attention_ops_match_pytorch_rocm():
    """The graph surface maps aten::_scaled_dot_product_flash_attention and its backward (what
    torch.compile makes of F.scaled_dot_product_attention on 16-bit tensors) to the fused
    kernels: same contract as PyTorch-ROCm's own ops, values against float64 autograd."""
    from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO as mapping
    aten = torch.ops.aten
    b, h, t = 2, 3, 200
    qkv = seeded((b, t, 3 * h * 64), seed=21, dtype=torch.bfloat16).cuda()
    q, k, v = (x.view(b, t, h, 64).transpose(1, 2) for x in qkv.split(h * 64, dim=2))
    dout = seeded((b, t, h, 64), seed=22, dtype=torch.bfloat16).cuda().transpose(1, 2)
    got = mapping[aten._scaled_dot_product_flash_attention](q, k, v, 0.0, True, False, scale=0.125)
    ref = aten._scaled_dot_product_flash_attention(q, k, v, 0.0, True, False, scale=0.125)
    assert len(got) == len(ref) == 9
    for g, r in zip(got, ref):
        if isinstance(r, torch.Tensor):
            assert g.shape == r.shape and g.dtype == r.dtype and g.device == r.device
            assert g.stride() == r.stride()
        else:
            assert g == r
    out64, lse64, *want = _float64_reference(q.cpu(), k.cpu(), v.cpu(), dout.cpu().transpose(1, 2), 0.125, True)
    assert np.abs(as64(got[0]) - out64.numpy()).max() <= 3e-2
    np.testing.assert_allclose(as64(got[1]), lse64.numpy(), rtol=0, atol=1e-4)
    np.testing.assert_allclose(as64(ref[1]), lse64.numpy(), rtol=0, atol=1e-3)  # same definition
    grads = mapping[aten._scaled_dot_product_flash_attention_backward](
        dout, q, k, v, got[0], got[1], None, None, t, t, 0.0, True, got[6], got[7], scale=0.125)
    ref_grads = aten._scaled_dot_product_flash_attention_backward(
        dout, q, k, v, ref[0], ref[1], None, None, t, t, 0.0, True, ref[6], ref[7], scale=0.125)
    for name, g, r, w in zip("qkv", grads, ref_grads, want):
        assert g.shape == r.shape and g.dtype == r.dtype and g.stride() == r.stride(), name
        big = w.abs().max().item()
        assert np.abs(as64(g) - w.numpy()).max() <= 2e-2 * big, name
    # and our backward accepts PyTorch-ROCm's forward results (same log-sum-exp definition)
    mixed = mapping[aten._scaled_dot_product_flash_attention_backward](
        dout, q, k, v, ref[0], ref[1], None, None, t, t, 0.0, True, ref[6], ref[7], scale=0.125)
    for name, g, w in zip("qkv", mixed, want):
        assert np.abs(as64(g) - w.numpy()).max() <= 2e-2 * w.abs().max().item(), name
    # dropout is PyTorch-ROCm's own op
    calls = []
    real = _ops().attention
    try:
        _ops().attention = lambda *a, **kw: calls.append(1) or real(*a, **kw)
        mapping[aten._scaled_dot_product_flash_attention](q, k, v, 0.5, True, False, scale=0.125)
    finally:
        _ops().attention = real
    assert not calls
