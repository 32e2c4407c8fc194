"""Whole models on the eager ``mojo`` device: the hot ops run on the HIP kernels, everything else
a GPT-2 forward or a greedy decode loop touches runs on the holders (reference:
mojo_device/mojo_device_aten_ops.py registers its ops one by one in the same way)."""

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mojo():
    from torch_mojo_backend import register_mojo_devices
    register_mojo_devices()
    return torch.device("mojo")


def test_demo_gpt2_forward_runs_eagerly_on_the_hip_kernels(mojo):
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch_mojo_backend.mojo_device.mojo_device_aten_ops import EAGER_CALL_COUNTERS
    model = build_gpt2_small(seed=0, n_layer=2)
    idx = seeded_tokens(2, 32, seed=0)
    with torch.no_grad():
        want_logits, want_next = model(idx)
    before = {k: v.call_count for k, v in EAGER_CALL_COUNTERS.items()}
    with torch.no_grad():
        logits, nxt = model.to(mojo)(idx.to(mojo))
    assert logits.device.type == "mojo"
    torch.testing.assert_close(logits.cpu(), want_logits, rtol=1e-4, atol=1e-4)
    assert torch.equal(nxt.cpu(), want_next)
    grew = {k for k, v in EAGER_CALL_COUNTERS.items() if v.call_count > before[k]}
    # every hot op of the forward went through its fast_aten_* twin
    # (eagerly, nn.Linear is aten::linear, F.softmax is aten::softmax.int and F.layer_norm is
    # aten::layer_norm, which skips the row statistics nobody reads without a gradient)
    for op in ("aten::linear", "aten::layer_norm", "aten::bmm", "aten::softmax.int",
               "aten::gelu", "aten::argmax"):
        assert op in grew, f"{op} did not run on the mojo device ({sorted(grew)})"


def test_hf_gpt2_greedy_generate_matches_cpu(mojo):
    transformers = pytest.importorskip("transformers")
    torch.manual_seed(0)
    model = transformers.GPT2LMHeadModel(transformers.GPT2Config(n_layer=2)).eval()
    ids = torch.randint(0, 50257, (4, 8))
    mask = torch.ones_like(ids)
    kw = dict(max_new_tokens=6, min_new_tokens=6, do_sample=False, pad_token_id=50256)
    with torch.no_grad():
        want = model.generate(ids, attention_mask=mask, **kw)
        got = model.to(mojo).generate(ids.to(mojo), attention_mask=mask.to(mojo), **kw)
    assert got.device.type == "mojo"
    assert torch.equal(got.cpu(), want)


def test_views_share_memory_and_inplace_ops_return_their_input(mojo):
    x = torch.arange(24, dtype=torch.float32).view(2, 3, 4).to(mojo)
    v = x.transpose(0, 2)[1:3]
    v.mul_(2.0)
    want = torch.arange(24, dtype=torch.float32).view(2, 3, 4)
    want.transpose(0, 2)[1:3].mul_(2.0)
    assert torch.equal(x.cpu(), want)
    y = x.add_(1.0)
    assert y is x
    parts = torch.split(x, 2, dim=2)
    assert all(p.device.type == "mojo" for p in parts)
    assert torch.equal(torch.cat(parts, dim=2).cpu(), want + 1.0)


def test_an_op_without_a_registration_still_raises(mojo):
    x = torch.rand(8).to(mojo)
    with pytest.raises(NotImplementedError):
        torch.erfinv(x)


def test_training_step_on_the_eager_device_matches_cpu_gradients(mojo):
    """Autograd over mojo tensors (reference mojo_device/mojo_device_autograd.py): PyTorch's own
    derivative formulas run on the wrapper tensors and reach the backward twins of the hot ops
    (linear_backward GEMMs, native_layer_norm_backward, gelu_backward, _log_softmax_backward_data)
    through the same PrivateUse1 registrations as the forward."""
    import copy

    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch_mojo_backend.mojo_device.mojo_device_aten_ops import EAGER_CALL_COUNTERS

    model = build_gpt2_small(seed=0, n_layer=2).train()
    idx = seeded_tokens(2, 32, seed=0)
    target = seeded_tokens(2, 32, seed=1)

    def loss_of(m, i, t):
        logits, _ = m(i)
        return torch.nn.functional.cross_entropy(logits.reshape(-1, logits.shape[-1]), t.reshape(-1))

    ref = copy.deepcopy(model)
    want = loss_of(ref, idx, target)
    want.backward()
    dev = copy.deepcopy(model).to(mojo)
    before = {k: v.call_count for k, v in EAGER_CALL_COUNTERS.items()}
    got = loss_of(dev, idx.to(mojo), target.to(mojo))
    got.backward()
    torch.testing.assert_close(got.detach().cpu(), want.detach(), rtol=1e-5, atol=1e-5)
    grew = {k for k, v in EAGER_CALL_COUNTERS.items() if v.call_count > before[k]}
    for op in ("aten::native_layer_norm_backward", "aten::gelu_backward", "aten::_log_softmax_backward_data"):
        assert op in grew, f"{op} did not run on the mojo device ({sorted(grew)})"
    checked = 0
    for (name, p), (_, q) in zip(dev.named_parameters(), ref.named_parameters()):
        assert p.grad is not None and p.grad.device.type == "mojo", name
        scale = q.grad.abs().max().item() + 1e-12
        err = (p.grad.cpu() - q.grad).abs().max().item()
        assert err <= 2e-4 * scale + 1e-7, f"{name}: gradient differs by {err} (scale {scale})"
        checked += 1
    assert checked >= 20
    # one SGD step on the device lowers the loss
    with torch.no_grad():
        for p in dev.parameters():
            p -= 0.5 * p.grad
    assert loss_of(dev, idx.to(mojo), target.to(mojo)).item() < got.item()


def test_sdpa_gradients_on_the_eager_device_come_from_the_fused_backward(mojo):
    """F.scaled_dot_product_attention with a gradient wanted, bf16 heads of 64: the autograd
    kernel routes to aten::_scaled_dot_product_flash_attention (fused forward + log-sum-exp) and
    PyTorch's derivative formula then calls the fused backward op; gradients match float64."""
    from torch_mojo_backend.mojo_device.mojo_device_aten_ops import EAGER_CALL_COUNTERS

    torch.manual_seed(3)
    b, h, t = 2, 3, 140
    qkv = torch.randn(b, t, 3 * h * 64).bfloat16()
    g = torch.randn(b, h, t, 64).bfloat16()

    def run(x, grad, dtype):
        x = x.to(dtype).requires_grad_(True)
        q, k, v = (y.view(b, t, h, 64).transpose(1, 2) for y in x.split(h * 64, dim=2))
        out = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
        (out * grad.to(dtype)).sum().backward()
        return out.detach(), x.grad

    want_out, want_grad = run(qkv, g, torch.float64)
    ops = ("aten::_scaled_dot_product_flash_attention", "aten::_scaled_dot_product_flash_attention_backward")
    before = [EAGER_CALL_COUNTERS[op].call_count for op in ops]
    got_out, got_grad = run(qkv.to(mojo), g.to(mojo), torch.bfloat16)
    assert [EAGER_CALL_COUNTERS[op].call_count - n for op, n in zip(ops, before)] == [1, 1]
    assert got_grad.device.type == "mojo" and got_grad.dtype == torch.bfloat16
    assert (got_out.cpu().double() - want_out).abs().max().item() <= 3e-2
    big = want_grad.abs().max().item()
    assert (got_grad.cpu().double() - want_grad).abs().max().item() <= 2e-2 * big
    # float32 heads keep the composed, differentiable route
    _, grad32 = run(qkv.to(mojo), g.to(mojo), torch.float32)
    assert (grad32.cpu().double() - want_grad).abs().max().item() <= 1e-4 * big


def test_cat_of_two_contiguous_tensors_is_one_launch_and_matches_torch(mojo):
    """The key/value-cache append of a decode step, and every alignment class of the row-append
    kernel (16-, 4-, 2- and 1-byte pieces); other inputs take PyTorch-ROCm's cat on the holders."""
    from torch_mojo_backend.eager_kernels import hip_ops

    calls = []
    real = hip_ops.cat2
    hip_ops.cat2 = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
    try:
        cases = [((4, 3, 10, 64), (4, 3, 1, 64), 2, torch.bfloat16),   # cache append
                 ((4, 3, 10, 64), (4, 3, 1, 64), -2, torch.float16),
                 ((5, 6), (5, 2), 1, torch.float32),                    # 4-byte pieces
                 ((5, 3), (5, 1), 1, torch.bfloat16),                   # 2-byte pieces
                 ((7, 3), (7, 2), 1, torch.uint8),                      # single bytes
                 ((2, 5), (3, 5), 0, torch.int64),                      # one row: plain append
                 ((3, 0, 4), (3, 2, 4), 1, torch.float32)]              # an empty first operand
        for sa, sb, dim, dtype in cases:
            a = (torch.randn(sa) * 10).to(dtype) if dtype.is_floating_point else torch.randint(0, 100, sa).to(dtype)
            b = (torch.randn(sb) * 10).to(dtype) if dtype.is_floating_point else torch.randint(0, 100, sb).to(dtype)
            got = torch.cat([a.to(mojo), b.to(mojo)], dim=dim)
            assert got.device.type == "mojo"
            assert torch.equal(got.cpu(), torch.cat([a, b], dim=dim)), (sa, sb, dim, dtype)
        assert len(calls) == len(cases)
        # three inputs, and a strided input: PyTorch-ROCm's cat
        x = torch.randn(4, 6)
        got = torch.cat([x.to(mojo), x.to(mojo), x.to(mojo)], dim=0)
        assert torch.equal(got.cpu(), torch.cat([x, x, x], dim=0))
        got = torch.cat([x.to(mojo).t(), x.to(mojo).t()], dim=1)
        assert torch.equal(got.cpu(), torch.cat([x.t(), x.t()], dim=1))
        assert len(calls) == len(cases)
    finally:
        hip_ops.cat2 = real


def test_lean_elementwise_and_split_match_torch(mojo):
    x, y = torch.randn(3, 8), torch.randn(3, 8)
    xm, ym = x.to(mojo), y.to(mojo)
    for got, want in ((xm + ym, x + y), (xm * ym, x * y), (xm - ym, x - y), (xm * 0.5, x * 0.5),
                      (2 + xm, 2 + x), (torch.pow(xm, 3.0), torch.pow(x, 3.0)), (torch.tanh(xm), torch.tanh(x)),
                      (torch.add(xm, ym, alpha=2), torch.add(x, y, alpha=2)),
                      (xm + ym[0], x + y[0]), (xm * torch.tensor(2.0), x * 2.0)):
        assert got.device.type == "mojo"
        torch.testing.assert_close(got.cpu(), want)
    parts = xm.split(3, dim=1)
    assert [tuple(p.shape) for p in parts] == [(3, 3), (3, 3), (3, 2)]
    for p, w in zip(parts, x.split(3, dim=1)):
        assert torch.equal(p.cpu(), w)


def test_layer_norm_without_gradient_skips_the_statistics(mojo):
    from torch_mojo_backend.eager_kernels import hip_ops

    seen = []
    real = hip_ops.layer_norm
    hip_ops.layer_norm = lambda *a, **k: (seen.append(k.get("need_stats", True)), real(*a, **k))[1]
    try:
        x, w, b = torch.randn(4, 5, 48), torch.randn(48), torch.randn(48)
        want = torch.nn.functional.layer_norm(x, (48,), w, b, 1e-5)
        with torch.no_grad():
            got = torch.nn.functional.layer_norm(x.to(mojo), (48,), w.to(mojo), b.to(mojo), 1e-5)
        torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-5)
        assert seen == [False]
        xg = x.to(mojo).requires_grad_(True)
        out = torch.nn.functional.layer_norm(xg, (48,), w.to(mojo), b.to(mojo), 1e-5)
        out.sum().backward()
        assert seen == [False, True] and xg.grad is not None
        xr = x.clone().requires_grad_(True)
        torch.nn.functional.layer_norm(xr, (48,), w, b, 1e-5).sum().backward()
        torch.testing.assert_close(xg.grad.cpu(), xr.grad, rtol=1e-4, atol=1e-5)
    finally:
        hip_ops.layer_norm = real
