"""Checks of a training step through ``mojo_backend``: the backward graph runs the backward twins
of the hot ops on the HIP kernels (reference: aten_functions.py:788-833, 2070-2102, 2323-2375) and
the parameter gradients match PyTorch CPU eager.

Run as ``python training_checks.py <check name>`` by tests/test_training.py, one fresh interpreter
per check: once ``register_mojo_devices()`` has run in a process, PyTorch takes PrivateUse1 for
the process's accelerator and its autograd engine can no longer run a backward pass over HIP
tensors (internal assert in torch/csrc/autograd/engine.cpp), so these checks must not share a
process with the eager-device tests."""

import sys

import torch
import torch.nn.functional as F


def _loss(model, idx, targets):
    logits, _ = model(idx)
    return F.cross_entropy(logits.view(-1, logits.shape[-1]), targets.view(-1))


def gpt2_training_step_gradients_match_cpu():
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO as mapping
    from torch_mojo_backend import mojo_backend

    idx, targets = seeded_tokens(2, 32, seed=0), seeded_tokens(2, 32, seed=1)
    ref = build_gpt2_small(seed=0, n_layer=2)
    ref_loss = _loss(ref, idx, targets)
    ref_loss.backward()

    model = build_gpt2_small(seed=0, n_layer=2).cuda()
    compiled = torch.compile(model, backend=mojo_backend)
    aten = torch.ops.aten
    watched = (aten.gelu_backward, aten._softmax_backward_data, aten.native_layer_norm_backward,
               aten.mm)
    before = {op: mapping[op].call_count for op in watched}
    loss = _loss(compiled, idx.cuda(), targets.cuda())
    loss.backward()
    torch.testing.assert_close(loss.cpu(), ref_loss, rtol=1e-5, atol=1e-5)
    for (name, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        assert p.grad is not None, name
        scale = q.grad.abs().max().item() + 1e-12
        assert (p.grad.cpu() - q.grad).abs().max().item() <= 2e-4 * scale, name
    grew = {op for op in watched if mapping[op].call_count > before[op]}
    # 2 layers: a GELU, a softmax and two layer norms per block plus the final layer norm, and
    # the weight / input gradient GEMMs
    assert grew == set(watched), f"not every backward twin ran: {grew}"


def training_graph_runs_the_fused_attention_forward_and_backward():
    """A bf16 training graph runs one fused attention forward and one fused attention backward
    per block (the partitioner replaces the chain and its backward nodes); a float32 graph, which
    the 16-bit kernels do not take, is split as PyTorch would. With a mask buffer that is not
    causal the same two steps run op by op. In every case the gradients match float64 autograd of
    the same weights."""
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.eager_kernels import hip_ops

    calls = {"fwd": 0, "bwd": 0}
    real_f, real_b = hip_ops.attention, hip_ops.attention_backward

    def fwd(*a, **k):
        calls["fwd"] += 1
        return real_f(*a, **k)

    def bwd(*a, **k):
        calls["bwd"] += 1
        return real_b(*a, **k)

    hip_ops.attention, hip_ops.attention_backward = fwd, bwd
    idx, targets = seeded_tokens(2, 64, seed=0), seeded_tokens(2, 64, seed=1)

    def punch_mask(model):
        for name, buf in model.named_buffers():
            if name.endswith("bias") and buf.dim() == 4:
                buf[..., 5, 40:50] = 1  # query 5 also sees ten later keys: not causal any more

    for dtype, bound, causal in ((torch.float32, 2e-4, True), (torch.bfloat16, 6e-2, True),
                                 (torch.bfloat16, 6e-2, False)):
        ref = build_gpt2_small(seed=0, n_layer=2).double()
        model = build_gpt2_small(seed=0, n_layer=2).to(dtype).cuda()
        if not causal:
            punch_mask(ref)
            punch_mask(model)
        _loss(ref, idx, targets).backward()
        calls["fwd"] = calls["bwd"] = 0
        loss = _loss(torch.compile(model, backend=mojo_backend), idx.cuda(), targets.cuda())
        fused = 2 if (dtype is torch.bfloat16 and causal) else 0
        assert calls == {"fwd": fused, "bwd": 0}, (dtype, causal, calls)
        loss.backward()
        assert calls == {"fwd": fused, "bwd": fused}, (dtype, causal, calls)
        for (name, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
            scale = q.grad.abs().max().item() + 1e-12
            err = (p.grad.double().cpu() - q.grad).abs().max().item()
            assert err <= bound * scale, (dtype, causal, name, err / scale)
        torch._dynamo.reset()


def attention_backward_follows_the_route_the_forward_took():
    """The mask buffer edited between forward and backward: the backward step takes the route the
    forward recorded in its log-sum-exp (all values: fused; no elements: op by op) and never
    asks about the buffer again. Fused forward + punched mask -> fused backward with the causal
    gradients; op-by-op forward + repaired mask -> op-by-op backward, finite gradients."""
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.eager_kernels import hip_ops

    calls = {"fwd": 0, "bwd": 0}
    real_f, real_b = hip_ops.attention, hip_ops.attention_backward

    def fwd(*a, **k):
        calls["fwd"] += 1
        return real_f(*a, **k)

    def bwd(*a, **k):
        calls["bwd"] += 1
        return real_b(*a, **k)

    hip_ops.attention, hip_ops.attention_backward = fwd, bwd
    idx, targets = seeded_tokens(2, 64, seed=0), seeded_tokens(2, 64, seed=1)

    def masks(model):
        return [b for n, b in model.named_buffers() if n.endswith("bias") and b.dim() == 4]

    ref = build_gpt2_small(seed=0, n_layer=2).double()
    _loss(ref, idx, targets).backward()
    model = build_gpt2_small(seed=0, n_layer=2).to(torch.bfloat16).cuda()
    loss = _loss(torch.compile(model, backend=mojo_backend), idx.cuda(), targets.cuda())
    assert calls == {"fwd": 2, "bwd": 0}
    for buf in masks(model):           # through .data: autograd's version check does not see it
        buf.data[..., 5, 40:50] = 1
    loss.backward()
    assert calls == {"fwd": 2, "bwd": 2}
    for (name, p), (_, q) in zip(model.named_parameters(), ref.named_parameters()):
        scale = q.grad.abs().max().item() + 1e-12
        err = (p.grad.double().cpu() - q.grad).abs().max().item()
        assert err <= 6e-2 * scale, (name, err / scale)
    torch._dynamo.reset()

    calls["fwd"] = calls["bwd"] = 0
    model = build_gpt2_small(seed=0, n_layer=2).to(torch.bfloat16).cuda()
    with torch.no_grad():
        for buf in masks(model):
            buf[..., 5, 40:50] = 1
    loss = _loss(torch.compile(model, backend=mojo_backend), idx.cuda(), targets.cuda())
    assert calls == {"fwd": 0, "bwd": 0}
    for buf in masks(model):
        buf.data[..., 5, 40:50] = 0
    loss.backward()
    assert calls == {"fwd": 0, "bwd": 0}
    assert all(torch.isfinite(p.grad).all().item() for p in model.parameters())
    torch._dynamo.reset()


def sdpa_training_graph_runs_the_fused_forward_and_backward():
    """F.scaled_dot_product_attention on bf16 tensors reaches a training graph as
    aten::_scaled_dot_product_flash_attention and its backward op: both run on the fused kernels
    and the gradients match float64 autograd of the same module."""
    from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO as mapping
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.eager_kernels import hip_ops

    class Block(torch.nn.Module):
        def __init__(self, heads=4):
            super().__init__()
            self.heads = heads
            self.qkv = torch.nn.Linear(heads * 64, 3 * heads * 64)
            self.proj = torch.nn.Linear(heads * 64, heads * 64)

        def forward(self, x):
            b, t, c = x.shape
            q, k, v = (y.view(b, t, self.heads, 64).transpose(1, 2) for y in self.qkv(x).split(c, dim=2))
            y = F.scaled_dot_product_attention(q, k, v, is_causal=True)
            return self.proj(y.transpose(1, 2).reshape(b, t, c))

    torch.manual_seed(0)
    ref = Block().double()
    x = torch.randn(2, 150, 256, dtype=torch.float64)
    g = torch.randn(2, 150, 256, dtype=torch.float64)
    xr = x.clone().requires_grad_(True)
    (ref(xr) * g).sum().backward()

    fused = {"fwd": 0, "bwd": 0}
    real_f, real_b = hip_ops.attention, hip_ops.attention_backward
    hip_ops.attention = lambda *a, **k: (fused.__setitem__("fwd", fused["fwd"] + 1), real_f(*a, **k))[1]
    hip_ops.attention_backward = lambda *a, **k: (fused.__setitem__("bwd", fused["bwd"] + 1), real_b(*a, **k))[1]
    model = Block().bfloat16().cuda()
    model.load_state_dict({k: v.bfloat16() for k, v in ref.state_dict().items()})
    aten = torch.ops.aten
    watched = (aten._scaled_dot_product_flash_attention, aten._scaled_dot_product_flash_attention_backward)
    before = [mapping[op].call_count for op in watched]
    xd = x.bfloat16().cuda().requires_grad_(True)
    (torch.compile(model, backend=mojo_backend)(xd) * g.bfloat16().cuda()).sum().backward()
    assert [mapping[op].call_count - n for op, n in zip(watched, before)] == [1, 1]
    assert fused == {"fwd": 1, "bwd": 1}, fused
    pairs = [("x", xd.grad, xr.grad)] + [(n, p.grad, q.grad) for (n, p), (_, q) in
                                         zip(model.named_parameters(), ref.named_parameters())]
    for name, got, want in pairs:
        scale = want.abs().max().item()
        err = (got.double().cpu() - want).abs().max().item()
        assert err <= 4e-2 * scale, (name, err / scale)


def one_sgd_step_lowers_the_loss():
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch_mojo_backend import mojo_backend

    idx, targets = seeded_tokens(4, 16, seed=2).cuda(), seeded_tokens(4, 16, seed=3).cuda()
    model = build_gpt2_small(seed=1, n_layer=1).cuda()
    compiled = torch.compile(model, backend=mojo_backend)
    opt = torch.optim.SGD(model.parameters(), lr=0.5)
    first = _loss(compiled, idx, targets)
    first.backward()
    opt.step()
    opt.zero_grad()
    second = _loss(compiled, idx, targets)
    assert second.item() < first.item()


def log_softmax_and_linear_backward_in_a_compiled_graph():
    from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO as mapping
    from torch_mojo_backend import mojo_backend

    torch.manual_seed(0)
    lin = torch.nn.Linear(96, 40)
    x = torch.randn(8, 17, 96)
    g = torch.randn(8, 17, 40)

    def fn(module, inp):
        return F.log_softmax(module(inp), dim=-1)

    xr = x.clone().requires_grad_(True)
    (fn(lin, xr) * g).sum().backward()
    want = (xr.grad, lin.weight.grad.clone(), lin.bias.grad.clone())
    lin.zero_grad()
    dev = torch.nn.Linear(96, 40).cuda()
    dev.load_state_dict(lin.state_dict())
    before = mapping[torch.ops.aten._log_softmax_backward_data].call_count
    xd = x.cuda().requires_grad_(True)
    (torch.compile(fn, backend=mojo_backend)(dev, xd) * g.cuda()).sum().backward()
    assert mapping[torch.ops.aten._log_softmax_backward_data].call_count > before
    for got, ref in zip((xd.grad, dev.weight.grad, dev.bias.grad), want):
        torch.testing.assert_close(got.cpu(), ref, rtol=1e-4, atol=1e-5)


def vocabulary_projection_backward_pads_its_gradient_once():
    """Both products of a 50257-wide projection's backward pass (the input gradient contracts
    over the vocabulary, the weight gradient has it as its transposed dimension) need the incoming
    gradient in rows of whole 16-byte vectors: one padded copy serves both, and the gradients
    still match float64 on the host."""
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.eager_kernels import hip_ops

    torch.manual_seed(0)
    rows, hidden, vocab = 1024, 256, 50257
    w = (torch.randn(vocab, hidden) * 0.05).bfloat16()
    x = torch.randn(rows, hidden).bfloat16()
    g = (torch.randn(rows, vocab) * 0.1).bfloat16()

    def fn(inp, weight, grad):
        return ((inp @ weight.t()) * grad).sum()

    copies = []
    plain_copy = hip_ops._pad_last_copy

    def counting(t, size):
        if t.numel() * t.element_size() >= hip_ops._PAD_REUSE_MIN_BYTES:
            copies.append((tuple(t.shape), size))
        return plain_copy(t, size)

    hip_ops._pad_last_copy = counting
    try:
        xd, wd = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
        torch.compile(fn, backend=mojo_backend)(xd, wd, g.cuda()).backward()
        torch.cuda.synchronize()
    finally:
        hip_ops._pad_last_copy = plain_copy
    assert copies == [((rows, vocab), 50304)], copies
    assert hip_ops.pad_reuse_active() is None
    want_dx = g.double() @ w.double()
    want_dw = g.double().t() @ x.double()
    for got, want in ((xd.grad, want_dx), (wd.grad, want_dw)):
        assert got.shape == want.shape and got.is_contiguous()
        err = (got.cpu().double() - want).norm() / want.norm()
        assert err < 4e-3, err


def cross_entropy_in_the_graph_sends_one_pass_back_to_the_logits():
    """A cross-entropy loss computed inside the compiled function, over a 50257-wide vocabulary:
    the backward graph's nll_loss_backward + _log_softmax_backward_data pair runs as one pass that
    writes rows of whole vectors, so neither product of the projection's backward pads the
    gradient again; ignored targets, mean and sum reductions, gradients against float64."""
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.eager_kernels import hip_ops

    torch.manual_seed(0)
    rows, hidden, vocab = 1024, 128, 50257
    w = (torch.randn(vocab, hidden) * 0.05).bfloat16()
    x = torch.randn(rows, hidden).bfloat16()
    t = torch.randint(0, vocab, (rows,))
    t[::7] = -100

    for reduction in ("mean", "sum"):
        def fn(inp, weight, target):
            return F.cross_entropy(inp @ weight.t(), target, reduction=reduction)

        fused, copies = [], []
        plain, plain_copy = hip_ops.nll_log_softmax_backward, hip_ops._pad_last_copy

        def counting(*args):
            fused.append(tuple(args[1].shape))
            return plain(*args)

        def counting_copy(tensor, size):
            if tensor.numel() * tensor.element_size() >= hip_ops._PAD_REUSE_MIN_BYTES:
                copies.append((tuple(tensor.shape), size))
            return plain_copy(tensor, size)

        hip_ops.nll_log_softmax_backward, hip_ops._pad_last_copy = counting, counting_copy
        try:
            xd, wd = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
            torch._dynamo.reset()
            loss = torch.compile(fn, backend=mojo_backend)(xd, wd, t.cuda())
            loss.backward()
            torch.cuda.synchronize()
        finally:
            hip_ops.nll_log_softmax_backward, hip_ops._pad_last_copy = plain, plain_copy
        assert fused == [(rows, vocab)], fused
        assert copies == [], copies
        assert hip_ops.pad_reuse_active() is None
        x64, w64 = x.double().requires_grad_(True), w.double().requires_grad_(True)
        want = F.cross_entropy(x64 @ w64.t(), t, reduction=reduction)
        want.backward()
        assert abs(float(loss) - float(want)) <= 2e-2 * abs(float(want))
        for got, ref in ((xd.grad, x64.grad), (wd.grad, w64.grad)):
            assert got.shape == ref.shape and got.is_contiguous()
            err = (got.cpu().double() - ref).norm() / ref.norm()
            assert err < 2e-2, (reduction, err)


def residual_gradient_joins_inside_the_layer_norm_backward():
    """Two decoder blocks: each native_layer_norm_backward of the backward graph also adds the
    gradient that by-passed its block and hands out the bias gradient of the projection in front
    of it (one pass instead of three). Every matrix gradient equals, bit for bit, that of the same
    graph run with the three ops apart; the vectors (bias and norm gradients, whose sums are
    added in another order) agree to rounding."""
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.eager_kernels import hip_ops

    idx, targets = seeded_tokens(4, 64, seed=0).cuda(), seeded_tokens(4, 64, seed=1).cuda()
    plain = hip_ops.layer_norm_backward_add
    for dtype in (torch.bfloat16, torch.float32):
        grads = {}
        for route in ("one pass", "apart"):
            taken = []

            def counting(*args):
                taken.append((args[6] is not None, args[7]))
                return plain(*args) if route == "one pass" else None

            hip_ops.layer_norm_backward_add = counting
            try:
                torch._dynamo.reset()
                model = build_gpt2_small(seed=0, n_layer=2).to(dtype).cuda()
                loss = _loss(torch.compile(model, backend=mojo_backend), idx, targets)
                loss.backward()
                torch.cuda.synchronize()
            finally:
                hip_ops.layer_norm_backward_add = plain
            # the final norm (sums only), then four norms with the by-passing gradient, the last
            # of which feeds no projection
            assert taken == [(False, True), (True, True), (True, True), (True, True), (True, False)], taken
            grads[route] = {n: p.grad.clone() for n, p in model.named_parameters()}
        for name, got in grads["one pass"].items():
            want = grads["apart"][name]
            if got.dim() >= 2:
                assert torch.equal(got, want), (dtype, name)
            else:
                scale = want.double().abs().max().item() + 1e-6
                tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
                assert (got.double() - want.double()).abs().max().item() <= tol * scale, (dtype, name)


def training_graphs_are_never_replayed():
    """TORCH_MOJO_BACKEND_HIP_GRAPH=1 records inference graphs only: the forward graph of a
    training step hands tensors to the backward pass, and neither of the two is ever replayed."""
    import os

    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.torch_compile_backend import compiler

    os.environ["TORCH_MOJO_BACKEND_HIP_GRAPH"] = "1"
    model = build_gpt2_small(seed=0, n_layer=1).bfloat16().cuda().train()
    compiled = torch.compile(model, backend=mojo_backend)
    before = dict(compiler.GRAPH_REPLAYS)
    for seed in range(3):
        logits, _ = compiled(seeded_tokens(2, 32, seed=seed).cuda())
        logits.float().sum().backward()
    torch.cuda.synchronize()
    assert compiler.GRAPH_REPLAYS == before, compiler.GRAPH_REPLAYS
    assert all(p.grad is not None for p in model.parameters())
    # the same module under no_grad is an inference graph: recorded at its second call
    with torch.no_grad():
        idx = seeded_tokens(2, 32, seed=5).cuda()
        outs = [compiled(idx)[0] for _ in range(4)]
    torch.cuda.synchronize()
    assert compiler.GRAPH_REPLAYS["recorded"] == before["recorded"] + 1
    assert all(torch.equal(outs[0], o) for o in outs[1:])


if __name__ == "__main__":
    import os

    os.environ["TORCH_MOJO_BACKEND_TESTING"] = "1"
    here = os.path.dirname(os.path.abspath(__file__))
    for p in (os.path.join(here, "..", "torch-max-backend_amd"), os.path.join(here, "..")):
        sys.path.insert(0, os.path.normpath(p))
    globals()[sys.argv[1]]()
    print("ok", sys.argv[1])
