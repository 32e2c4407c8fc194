"""End-to-end: the GPT-2-small-shaped forward through torch.compile(backend=mojo_backend) on the
HIP kernels, against PyTorch CPU eager float32 of the same seeded module (the reference's
check_functions_are_equivalent, torch_mojo_backend/testing.py:139-166)."""

import pytest
import torch

from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
from helpers import seeded

pytestmark = pytest.mark.gpu


def _hot_counts():
    from torch_mojo_backend import aten_functions as af
    return {f.__name__: f.call_count for f in (af.aten_addmm, af.aten_mm, af.aten_bmm,
                                               af.aten__softmax, af.aten_native_layer_norm,
                                               af.aten_argmax, af.aten_gelu)}


def test_gpt2_small_fp32_batch1_seq128_matches_cpu_eager():
    """Workload: 12 layers, d 768, 12 heads, B=1, T=128, float32, seed 0."""
    from torch_mojo_backend import mojo_backend

    model = build_gpt2_small(seed=0)
    idx = seeded_tokens(1, 128, seed=0)
    with torch.no_grad():
        want_logits, want_next = model(idx)
    gpu_model = build_gpt2_small(seed=0).to("cuda")
    compiled = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)
    before = _hot_counts()
    with torch.no_grad():
        logits, nxt = compiled(idx.to("cuda"))
    after = _hot_counts()
    assert logits.shape == (1, 128, 50257) and logits.dtype == torch.float32
    # every hot op of the graph went through the HIP mapping functions
    # (of the 48 addmm, c_fc's 12 run fused with their gelu and the 24 projections in front of a
    # residual add run fused with that add; those steps launch the GEMM kernel directly)
    assert after["aten_addmm"] - before["aten_addmm"] == 12
    assert after["aten_bmm"] - before["aten_bmm"] == 24
    # mul + masked_fill + _softmax run as one fused step that launches the kernel directly
    assert after["aten__softmax"] - before["aten__softmax"] == 0
    assert after["aten_native_layer_norm"] - before["aten_native_layer_norm"] == 25
    assert after["aten_mm"] - before["aten_mm"] == 1
    assert after["aten_argmax"] - before["aten_argmax"] == 1
    # float32 end to end: 25 layer norms and 97 GEMMs deep, so a few 1e-5 relative
    torch.testing.assert_close(logits.cpu(), want_logits, rtol=1e-4, atol=1e-4)
    # argmax is exact on the backend's own logits ...
    assert torch.equal(nxt.cpu(), torch.argmax(logits[:, -1, :], dim=-1).cpu())
    # ... and agrees with the oracle wherever the oracle's top-2 margin exceeds the tolerance
    top2 = want_logits[:, -1, :].topk(2, dim=-1).values
    if (top2[:, 0] - top2[:, 1]).min() > 2e-4:
        assert torch.equal(nxt.cpu(), want_next)


def test_gpt2_small_bf16_logits_vs_fp32_oracle():
    """bf16 weights/activations on the GPU vs float32 CPU eager on the same bf16-rounded weights:
    max-abs logit error <= 2e-2, the bound the workload definition states.

    What makes the bound reachable is the graph executor, not a kernel: a bf16 pipeline that
    rounds the residual stream to bf16 after each of its 24 adds lands at 2.9e-2 .. 3.6e-2
    (PyTorch-ROCm's bf16 eager run and PyTorch's CPU bf16 eager run of the same module, both
    printed below, as well as this backend with TORCH_MOJO_BACKEND_ROUND_LIKE_UNFUSED=1). The
    executor keeps that stream in float32 between the fused residual GEMMs and the layer norms
    that read it, and evaluates fused GELU / residual epilogues in float32 up to their one cast."""
    from torch_mojo_backend import mojo_backend

    model = build_gpt2_small(seed=0)
    model = model.to(torch.bfloat16).to(torch.float32)   # weights rounded to bf16, math in fp32
    idx = seeded_tokens(2, 256, seed=1)
    with torch.no_grad():
        want_logits, _ = model(idx)
        cpu_bf16_logits, _ = build_gpt2_small(seed=0).to(torch.bfloat16)(idx)
    gpu_model = build_gpt2_small(seed=0).to(torch.bfloat16).to("cuda")
    with torch.no_grad():
        vendor_logits, _ = gpu_model(idx.to("cuda"))
    compiled = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)
    with torch.no_grad():
        logits, nxt = compiled(idx.to("cuda"))
    assert logits.dtype == torch.bfloat16
    err = (logits.float().cpu() - want_logits).abs()
    vendor_err = (vendor_logits.float().cpu() - want_logits).abs()
    cpu16_err = (cpu_bf16_logits.float() - want_logits).abs()
    vs_cpu16 = (logits.float().cpu() - cpu_bf16_logits.float()).abs()
    print(f"max-abs logit error vs the float32 model: ours {err.max().item():.4f} (mean "
          f"{err.mean().item():.5f}); PyTorch-ROCm bf16 eager {vendor_err.max().item():.4f} "
          f"({vendor_err.mean().item():.5f}); PyTorch CPU bf16 eager {cpu16_err.max().item():.4f} "
          f"({cpu16_err.mean().item():.5f}); ours vs CPU bf16 eager {vs_cpu16.max().item():.4f}")
    assert err.max().item() <= 2e-2
    assert err.mean().item() <= 3e-3
    # two bf16 pipelines differ from each other by more than either differs from float32 (their
    # storage roundings are independent): the reference's same-dtype check against CPU eager
    # (torch_mojo_backend/testing.py:186-229) holds at its own bf16 tolerance, not at 2e-2
    assert vs_cpu16.max().item() <= 1.25 * cpu16_err.max().item() + 1e-2
    assert torch.equal(nxt.cpu(), torch.argmax(logits[:, -1, :], dim=-1).cpu())


def test_gpt2_small_bf16_second_batch_size_runs_the_symbolic_graph():
    """A compiled module called with a second batch size is retraced with a symbolic batch
    dimension: the plans made at build time then hold symbols where the first graph held numbers,
    and every step has to take its sizes from the tensors it is handed. Both sizes, and the first
    one again, give the logits of the graph compiled for that size alone."""
    from torch_mojo_backend import mojo_backend

    gpu_model = build_gpt2_small(seed=0).to(torch.bfloat16).to("cuda")
    torch._dynamo.reset()
    compiled = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)
    got = {}
    with torch.no_grad():
        for batch in (2, 3, 2):
            idx = seeded_tokens(batch, 128, seed=batch).to("cuda")
            got[batch] = (idx, compiled(idx)[0])
    for batch, (idx, logits) in got.items():
        torch._dynamo.reset()
        alone = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)
        with torch.no_grad():
            want = alone(idx)[0]
        assert logits.shape == (batch, 128, 50257)
        assert (logits.float() - want.float()).abs().max().item() <= 2e-2
    torch._dynamo.reset()


@pytest.mark.parametrize("dynamic", [None, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_layer_gpt2_with_changing_batch_and_sequence_length(dtype, dynamic):
    """One compiled module, seven (batch, sequence) shapes in a row, with the shapes left to
    dynamo (static first, symbolic after the first change) and declared dynamic from the start:
    every fused step and the attention rewrite take their sizes from the tensors at run time.
    Reference: the same module in PyTorch-ROCm eager (same dtype), float32 to 1e-4, bf16 to the
    spread two bf16 pipelines show on this model."""
    from torch_mojo_backend import mojo_backend

    model = build_gpt2_small(seed=0, n_layer=2).to(dtype).to("cuda")
    torch._dynamo.reset()
    compiled = torch.compile(model, backend=mojo_backend, dynamic=dynamic)
    for batch, seq in ((2, 128), (3, 128), (3, 256), (1, 64), (4, 100), (2, 1), (5, 77)):
        idx = seeded_tokens(batch, seq, seed=1000 * batch + seq).to("cuda")
        with torch.no_grad():
            got, nxt = compiled(idx)
            want, _ = model(idx)
        assert got.shape == (batch, seq, 50257) and got.dtype == dtype
        err = (got.float() - want.float()).abs().max().item()
        assert err <= (1e-4 if dtype == torch.float32 else 4e-2), (batch, seq, err)
        assert torch.equal(nxt, torch.argmax(got[:, -1, :], dim=-1))
    torch._dynamo.reset()


def test_gpt2_small_bf16_bit_identical_mode_matches_the_vendor_pipeline(monkeypatch):
    """TORCH_MOJO_BACKEND_ROUND_LIKE_UNFUSED=1: every tensor of the graph is rounded where the
    unfused kernels would have stored it; the logit error is then that of any bf16 pipeline."""
    from torch_mojo_backend import mojo_backend

    monkeypatch.setenv("TORCH_MOJO_BACKEND_ROUND_LIKE_UNFUSED", "1")
    model = build_gpt2_small(seed=0).to(torch.bfloat16).to(torch.float32)
    idx = seeded_tokens(2, 256, seed=1)
    with torch.no_grad():
        want_logits, _ = model(idx)
    gpu_model = build_gpt2_small(seed=0).to(torch.bfloat16).to("cuda")
    with torch.no_grad():
        vendor_logits, _ = gpu_model(idx.to("cuda"))
        logits, _ = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)(idx.to("cuda"))
    err = (logits.float().cpu() - want_logits).abs()
    vendor_err = (vendor_logits.float().cpu() - want_logits).abs()
    print(f"bit-identical mode: ours {err.max().item():.4f}, PyTorch-ROCm {vendor_err.max().item():.4f}")
    assert err.max().item() <= 1.1 * vendor_err.max().item()
    assert err.max().item() <= 3.6e-2
    assert err.mean().item() <= 5e-3


def test_gpt2_small_bf16_full_size_graph_routes_every_hot_op():
    """The benchmark configuration itself (B=32, T=1024, bf16): every GEMM, layer norm, the
    attention and the argmax run on the HIP kernels (call counts of the mapping functions and of
    the fused steps), the argmax is exact on the graph's own logits, batch rows 0 and 31 are within
    2e-2 (max-abs) of the float32 CPU model run on those rows alone, and rows sampled from the
    logits equal those of the same graph without the attention rewrite up to the reordered
    storage roundings."""
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.torch_compile_backend import compiler
    import os

    B, T = 32, 1024
    gpu_model = build_gpt2_small(seed=0).to(torch.bfloat16).to("cuda")
    idx = seeded_tokens(B, T, seed=0).to("cuda")
    hip_ops = compiler.aten_functions.hip_ops
    counts = {"gemm": 0, "attention": 0, "layer_norm": 0, "argmax": 0, "embedding": 0, "residual": 0,
              "gelu_epilogue": 0, "wide_out": 0, "wide_ln": 0}
    real = {n: getattr(hip_ops, n) for n in ("gemm", "attention", "layer_norm", "argmax", "embedding")}

    def gemm(a, b, bias=None, epilogue=0, residual=None, out_dtype=None, round_like_unfused=False):
        counts["gemm"] += 1
        counts["residual"] += residual is not None
        counts["gelu_epilogue"] += epilogue != 0
        counts["wide_out"] += out_dtype is torch.float32
        return real["gemm"](a, b, bias, epilogue, residual, out_dtype, round_like_unfused)

    def layer_norm(x, shape, w, b, eps, need_stats=True, out_dtype=None):
        counts["layer_norm"] += 1
        counts["wide_ln"] += x.dtype == torch.float32 and out_dtype == torch.bfloat16
        return real["layer_norm"](x, shape, w, b, eps, need_stats, out_dtype)

    def counted(name):
        def run(*a, **k):
            counts[name] += 1
            return real[name](*a, **k)
        return run

    patched = {"gemm": gemm, "layer_norm": layer_norm, "attention": counted("attention"),
               "argmax": counted("argmax"), "embedding": counted("embedding")}
    for n, f in patched.items():
        setattr(hip_ops, n, f)
    try:
        with torch.no_grad():
            logits, nxt = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)(idx)
    finally:
        for n, f in real.items():
            setattr(hip_ops, n, f)
    assert logits.shape == (B, T, 50257) and logits.dtype == torch.bfloat16
    # per layer: c_attn, c_proj (+residual), c_fc (+gelu), c_proj (+residual); plus lm_head
    assert counts["gemm"] == 12 * 4 + 1
    assert counts["residual"] == 24 and counts["gelu_epilogue"] == 12
    assert counts["wide_out"] == 24 and counts["wide_ln"] == 24       # float32 residual stream
    assert counts["attention"] == 12 and counts["layer_norm"] == 25
    assert counts["argmax"] == 1 and counts["embedding"] == 2
    assert torch.equal(nxt, torch.argmax(logits[:, -1, :].float(), dim=-1))
    # The tolerance the workload states, at the workload's own sequence length: batch rows are
    # independent, so the float32 CPU model (bf16-rounded weights) run on single rows of the batch
    # is the reference for those rows of the B = 32 graph (the reference's harness compares whole
    # outputs with the CPU run of the same module, torch_mojo_backend/testing.py:186-229).
    ref_model = build_gpt2_small(seed=0).to(torch.bfloat16).to(torch.float32)
    worst = 0.0
    for b in (0, 31):
        with torch.no_grad():
            want, want_next = ref_model(idx[b:b + 1].cpu())
        err = (logits[b].float().cpu() - want[0]).abs()
        print(f"B=32 T=1024 batch row {b}: max-abs logit error vs the float32 model "
              f"{err.max().item():.4f} (mean {err.mean().item():.5f})")
        worst = max(worst, err.max().item())
        assert err.mean().item() <= 3e-3
        top2 = want[0, -1].topk(2).values
        if (top2[0] - top2[1]).item() > 4e-2:
            assert nxt[b].item() == want_next[0].item()
    assert worst <= 2e-2
    rows = [(0, 0), (0, 1023), (7, 511), (31, 0), (31, 1023)]
    picked = torch.stack([logits[b, t] for b, t in rows]).float()
    del logits
    os.environ["TORCH_MOJO_BACKEND_NO_ATTENTION_FUSION"] = "1"
    try:
        torch.compiler.reset()
        with torch.no_grad():
            plain, nxt_plain = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)(idx)
    finally:
        del os.environ["TORCH_MOJO_BACKEND_NO_ATTENTION_FUSION"]
    other = torch.stack([plain[b, t] for b, t in rows]).float()
    diff = (picked - other).abs()
    assert diff.max().item() <= 3e-2 and diff.mean().item() <= 2.0 ** -8
    assert (nxt == nxt_plain).float().mean().item() >= 0.9


def test_fusion_is_bit_identical_to_unfused(monkeypatch):
    """With TORCH_MOJO_BACKEND_ROUND_LIKE_UNFUSED=1 the addmm->gelu, addmm->add and
    mul+masked_fill+softmax rewrites must not change a single bit of the logits (the attention
    rewrite reorders roundings and is checked to a tolerance below)."""
    from torch_mojo_backend import mojo_backend

    monkeypatch.setenv("TORCH_MOJO_BACKEND_NO_ATTENTION_FUSION", "1")
    monkeypatch.setenv("TORCH_MOJO_BACKEND_ROUND_LIKE_UNFUSED", "1")
    gpu_model = build_gpt2_small(seed=0, n_layer=2).to(torch.bfloat16).to("cuda")
    idx = seeded_tokens(2, 64, seed=2).to("cuda")
    with torch.no_grad():
        fused, _ = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)(idx)
    torch.compiler.reset()
    monkeypatch.setenv("TORCH_MOJO_BACKEND_NO_FUSION", "1")
    with torch.no_grad():
        unfused, _ = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)(idx)
    assert torch.equal(fused, unfused)


class _Scores(torch.nn.Module):
    def __init__(self, block, causal):
        super().__init__()
        mask = torch.tril(torch.ones(block, block))
        if not causal:
            mask = (torch.rand(block, block, generator=torch.Generator().manual_seed(3)) > 0.4).float()
            mask[:, 0] = 1.0
        self.register_buffer("bias", mask.view(1, 1, block, block), persistent=False)

    def forward(self, q, k):
        t = q.shape[-2]
        att = (q @ k.transpose(-2, -1)) * (1.0 / 8.0)
        att = att.masked_fill(self.bias[:, :, :t, :t] == 0, float("-inf"))
        return torch.softmax(att, dim=-1)


@pytest.mark.parametrize("causal", [True, False])
def test_masked_softmax_fusion_on_device(causal, monkeypatch):
    """Causal buffer -> one fused kernel; any other mask -> the unfused ops inside the same
    step. Either way the result has the bits of the unfused graph."""
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.torch_compile_backend import compiler

    model = _Scores(128, causal).to("cuda").eval()
    q = seeded((2, 4, 96, 64), seed=1, dtype=torch.bfloat16).to("cuda")
    k = seeded((2, 4, 96, 64), seed=2, dtype=torch.bfloat16).to("cuda")
    calls = []
    real = compiler.aten_functions.hip_ops.softmax_scaled
    monkeypatch.setattr(compiler.aten_functions.hip_ops, "softmax_scaled",
                        lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    with torch.no_grad():
        fused = torch.compile(model, backend=mojo_backend, fullgraph=True)(q, k)
    assert bool(calls) == causal
    torch.compiler.reset()
    monkeypatch.setenv("TORCH_MOJO_BACKEND_NO_FUSION", "1")
    with torch.no_grad():
        unfused = torch.compile(model, backend=mojo_backend, fullgraph=True)(q, k)
    assert torch.equal(fused, unfused)
    want = model.float().cpu()(q.float().cpu(), k.float().cpu())
    assert (fused.float().cpu() - want).abs().max().item() <= 2e-2


def test_causal_verdict_follows_the_buffer_not_its_address():
    from torch_mojo_backend.torch_compile_backend import compiler

    x = torch.zeros(1, 1, 64, 64, device="cuda")
    mask = torch.tril(torch.ones(1, 1, 64, 64, device="cuda"))
    assert compiler._causal_q_len(mask, (), x) == 64
    assert compiler._causal_q_len(mask, (), x) == 64            # cached
    mask[0, 0, 3, 40] = 1.0                                      # in-place edit: no longer causal
    assert compiler._causal_q_len(mask, (), x) == 0
    addr = mask.data_ptr()
    del mask
    other = torch.ones(1, 1, 64, 64, device="cuda")              # likely the same block again
    assert compiler._causal_q_len(other, (), x) == 0
    assert other.data_ptr() == addr or True
    # a sliced view of a larger causal buffer
    big = torch.tril(torch.ones(1, 1, 128, 128, device="cuda"))
    assert compiler._causal_q_len(big, ((2, 0, 64, 1), (3, 0, 64, 1)), x) == 64
    assert compiler._causal_q_len(big, ((2, 0, 64, 1), (3, 1, 65, 1)), x) == 0


def test_a_running_step_never_compares_mask_values(monkeypatch):
    """check=False is how every step of a running graph asks: the answer comes from verdicts
    taken while the graph was built (exact slices, or any slice from the origin of a buffer
    that is causal as a whole: the sizes of a graph with dynamic shapes), and a buffer without
    a valid verdict (never seen, or edited since) gives 0 = run the unfused ops. No comparison,
    hence no synchronisation, on that path."""
    from torch_mojo_backend.torch_compile_backend import compiler

    mask = torch.tril(torch.ones(1, 1, 128, 128, device="cuda"))
    x = (64, 64)
    origin = ((2, 0, 64, 1), (3, 0, 64, 1))
    assert compiler._causal_q_len(mask, origin, x, check=False) == 0      # never seen
    compiler._take_causal_verdict(mask, None, None)                        # build time
    monkeypatch.setattr(compiler, "_is_causal", lambda *a: pytest.fail("values compared in a step"))
    assert compiler._causal_q_len(mask, origin, x, check=False) == 64
    assert compiler._causal_q_len(mask, ((2, 0, 2 ** 63 - 1, 1), (3, 0, 2 ** 63 - 1, 1)), (128, 128),
                                  check=False) == 128
    assert compiler._causal_q_len(mask, ((2, 0, 96, 1), (3, 0, 96, 1)), (96, 96), check=False) == 96
    assert compiler._causal_q_len(mask, ((2, 0, 64, 1), (3, 1, 65, 1)), x, check=False) == 0
    assert compiler._causal_q_len(mask, ((2, 0, 64, 2), (3, 0, 64, 1)), (32, 64), check=False) == 0
    assert compiler._causal_q_len(mask, origin, (64, 32), check=False) == 0  # sizes do not match
    mask[0, 0, 3, 40] = 1.0                                                 # edited: verdict void
    assert compiler._causal_q_len(mask, origin, x, check=False) == 0
    # a host buffer's verdict travels with each device copy made for a call
    monkeypatch.undo()
    host = torch.tril(torch.ones(1, 1, 32, 32))
    compiler._take_causal_verdict(host, ((2, 0, 16, 1), (3, 0, 16, 1)), (16, 16))
    copy = compiler._on_device(host, torch.device("cuda", 0))
    monkeypatch.setattr(compiler, "_is_causal", lambda *a: pytest.fail("values compared in a step"))
    assert compiler._causal_q_len(copy, ((2, 0, 16, 1), (3, 0, 16, 1)), (16, 16), check=False) == 16
    assert compiler._causal_q_len(copy, ((2, 0, 8, 1), (3, 0, 8, 1)), (8, 8), check=False) == 8


def test_attention_fusion_stays_within_the_storage_rounding(monkeypatch):
    """Whole-block attention in one kernel against the same graph without that rewrite:
    bf16 logits differ by the reordered roundings only."""
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.torch_compile_backend import compiler

    gpu_model = build_gpt2_small(seed=0, n_layer=2).to(torch.bfloat16).to("cuda")
    idx = seeded_tokens(2, 256, seed=2).to("cuda")
    calls = []
    real = compiler.aten_functions.hip_ops.attention
    monkeypatch.setattr(compiler.aten_functions.hip_ops, "attention",
                        lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    with torch.no_grad():
        fused, _ = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)(idx)
    assert len(calls) == 2                      # one launch per layer
    torch.compiler.reset()
    monkeypatch.setenv("TORCH_MOJO_BACKEND_NO_ATTENTION_FUSION", "1")
    with torch.no_grad():
        plain, _ = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)(idx)
    assert len(calls) == 2
    # Neither is "the" answer: measure both against the float32 CPU model on the same (bf16-
    # rounded) weights. The fused graph must be no further from it than the unfused one.
    ref_model = build_gpt2_small(seed=0, n_layer=2).to(torch.bfloat16).float()
    with torch.no_grad():
        want, _ = ref_model(idx.cpu())
    err_fused = (fused.float().cpu() - want).abs()
    err_plain = (plain.float().cpu() - want).abs()
    print(f"attention fusion: max-abs error fused {err_fused.max().item():.4f}, unfused "
          f"{err_plain.max().item():.4f}")
    assert err_fused.max().item() <= 2e-2
    assert err_fused.mean().item() <= 1.1 * err_plain.mean().item() + 1e-4
    # and the two agree to about one bf16 spacing of a logit of magnitude ~1 (2^-7) on average
    diff = (fused.float() - plain.float()).abs()
    assert diff.max().item() <= 4e-2 and diff.mean().item() <= 2.0 ** -7


def test_attention_fusion_falls_back_for_a_non_causal_buffer(monkeypatch):
    """Same graph, but the mask buffer is not lower-triangular: the fused step must run the
    unfused chain and give the unfused graph's bits."""
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.torch_compile_backend import compiler

    monkeypatch.setenv("TORCH_MOJO_BACKEND_ROUND_LIKE_UNFUSED", "1")
    gpu_model = build_gpt2_small(seed=0, n_layer=1).to(torch.bfloat16).to("cuda")
    for block in gpu_model.transformer.h:
        block.attn.bias[0, 0, 5, 40] = 1.0      # one key above the diagonal becomes visible
    idx = seeded_tokens(1, 128, seed=3).to("cuda")
    calls = []
    real = compiler.aten_functions.hip_ops.attention
    monkeypatch.setattr(compiler.aten_functions.hip_ops, "attention",
                        lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    with torch.no_grad():
        fused, _ = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)(idx)
    assert not calls
    torch.compiler.reset()
    monkeypatch.setenv("TORCH_MOJO_BACKEND_NO_FUSION", "1")
    with torch.no_grad():
        plain, _ = torch.compile(gpu_model, backend=mojo_backend, fullgraph=True)(idx)
    assert torch.equal(fused, plain)
