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
    # (eagerly, nn.Linear is aten::linear and F.softmax is aten::softmax.int; nothing decomposes)
    for op in ("aten::linear", "aten::native_layer_norm", "aten::bmm", "aten::softmax.int",
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
