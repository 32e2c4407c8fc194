"""The eager ``mojo`` device surface.

GPU part: tensors move to ``mojo``, the hot aten ops dispatch through PrivateUse1 to
``fast_aten_*`` and the HIP kernels, results match PyTorch CPU eager (the reference's
``check_outputs``). Host part (no GPU): the NOT_HANDLED ladder of ``aten_fast`` with stand-in
tensors, the reference's own fake-backend pattern (tests/test_tensor_spec_oom.py:14-143)."""

import types

import pytest
import torch

import torch_mojo_backend
from torch_mojo_backend import register_mojo_devices
from torch_mojo_backend.eager_kernels import aten_fast
from torch_mojo_backend.mojo_device import mojo_device_aten_ops as reg

register_mojo_devices()


# ---------------------------------------------------------------------------
# host logic (runs anywhere)
# ---------------------------------------------------------------------------
def _fake(shape, dtype=torch.float32, device="cuda:0"):
    numel = 1
    for s in shape:
        numel *= s
    return types.SimpleNamespace(_shape=tuple(shape), _dtype=dtype, _numel=numel,
                                 _device=torch.device(device), _holder=None)


@pytest.fixture()
def fake_backend(monkeypatch):
    """aten_fast sees stand-in tensors; any kernel launch or wrap is recorded, not executed."""
    launched = []
    monkeypatch.setattr(aten_fast, "_t", lambda x: x if isinstance(x, types.SimpleNamespace) else None)
    monkeypatch.setattr(aten_fast, "_wrap", lambda holder: ("wrapped", holder))
    monkeypatch.setattr(aten_fast.hip_ops, "gemm_if_planned", lambda *a, **k: None)  # nothing planned yet
    for name in ("gemm", "softmax", "layer_norm", "reduce", "argmax", "gelu"):
        monkeypatch.setattr(aten_fast.hip_ops, name,
                            lambda *a, _n=name, **k: launched.append(_n) or (_n, _n, _n))
    return launched


def test_registration_helpers_collect_the_hot_ops():
    names = [n for n, _ in reg._aten_ops_registry]
    for op in ("aten::mm", "aten::addmm", "aten::bmm", "aten::linear", "aten::_softmax",
               "aten::softmax.int", "aten::_log_softmax", "aten::native_layer_norm",
               "aten::sum.dim_IntList", "aten::mean", "aten::mean.dim", "aten::amax",
               "aten::argmax", "aten::gelu"):
        assert op in names
        assert hasattr(reg.EAGER_CALL_COUNTERS[op], "call_count")
    for name in ("fast_aten_mm", "fast_aten_addmm", "fast_aten_linear", "fast_aten_bmm",
                 "fast_aten__softmax", "fast_aten_softmax", "fast_aten__log_softmax",
                 "fast_aten_native_layer_norm", "fast_aten_sum", "fast_aten_mean",
                 "fast_aten_amax", "fast_aten_argmax"):
        assert hasattr(getattr(aten_fast, name), "call_count")
    assert torch_mojo_backend.TorchMojoTensor is not None


def test_not_handled_becomes_a_named_not_implemented_error():
    impl = reg._eager_impl("fast_aten_mm", "aten::mm")
    with pytest.raises(NotImplementedError) as info:
        impl(torch.randn(2, 3), torch.randn(3, 2))
    text = str(info.value)
    assert "aten::mm is not supported by mojo eager mode for these inputs" in text
    assert "(2, 3):torch.float32:cpu" in text


def test_addmm_rules(fake_backend):
    a, b = _fake((4, 8)), _fake((8, 6))
    assert aten_fast.fast_aten_addmm(_fake((6,)), a, b) != aten_fast.NOT_HANDLED
    assert fake_backend == ["gemm"]
    assert aten_fast.fast_aten_addmm(_fake((6,)), a, b, beta=0.5) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_addmm(_fake((6,)), a, b, alpha=2) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_addmm(_fake((5,)), a, b) is aten_fast.NOT_HANDLED          # bad bias
    assert aten_fast.fast_aten_addmm(_fake((6,), torch.bfloat16), a, b) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_addmm(_fake((6,)), a, _fake((7, 6))) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_addmm(_fake((6,)), a, _fake((8, 6), device="cuda:1")) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_mm(_fake((4, 8), torch.int64), _fake((8, 6), torch.int64)) is aten_fast.NOT_HANDLED
    assert fake_backend == ["gemm"]  # nothing was launched for any rejected call


def test_softmax_rules(fake_backend):
    x = _fake((4, 8))
    assert aten_fast.fast_aten__softmax(x, -1) != aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten__softmax(x, 2) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten__softmax(_fake((0, 8)), -1) is aten_fast.NOT_HANDLED        # numel == 0
    assert aten_fast.fast_aten__softmax(_fake((4, 8), torch.int64), -1) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten__softmax(x, -1, True) is aten_fast.NOT_HANDLED              # fp32 + half_to_float
    assert aten_fast.fast_aten__softmax(_fake((4, 8), torch.bfloat16), -1, True) != aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten__log_softmax(_fake((4, 8), torch.bfloat16), -1, True) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten__log_softmax(_fake((4, 8), torch.float16), -1, True) != aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_softmax(x, -1, torch.float32) is aten_fast.NOT_HANDLED      # dtype= unsupported


def test_layer_norm_rejects_metadata_before_materializing(fake_backend):
    x = _fake((2, 3, 8))
    ok = aten_fast.fast_aten_native_layer_norm(x, [8], _fake((8,)), _fake((8,)), 1e-5)
    assert ok != aten_fast.NOT_HANDLED and fake_backend == ["layer_norm"]
    bad = [
        (x, [7], None, None),                                   # trailing dims do not match
        (x, [], None, None),                                    # k < 1
        (x, [8], _fake((7,)), None),                            # weight shape
        (x, [8], _fake((8,), torch.bfloat16), None),            # weight dtype
        (x, [8], None, _fake((8,), device="cuda:1")),           # bias device
        (_fake((0, 8)), [8], None, None),                       # empty
        (_fake((2, 8), torch.int32), [8], None, None),          # dtype
    ]
    for inp, shape, w, b in bad:
        assert aten_fast.fast_aten_native_layer_norm(inp, shape, w, b, 1e-5) is aten_fast.NOT_HANDLED
    assert fake_backend == ["layer_norm"]


def test_reduce_dim_rules():
    n = aten_fast._norm_reduce_dims
    assert n(None, 3, True) == [0, 1, 2]
    assert n([], 3, True) == [0, 1, 2] and n([], 3, False) == []
    assert n(-1, 3, True) == [2] and n([2, 0], 3, True) == [0, 2]
    assert n([0, 0], 3, True) is None and n([3], 3, True) is None and n([True], 3, True) is None
    assert n("x", 3, True) is None
    assert aten_fast._reduced_shape((4, 5, 6), [0, 2], True) == (1, 5, 1)
    assert aten_fast._reduced_shape((4, 5, 6), [0, 2], False) == (5,)


def test_reduction_dtype_rules(fake_backend):
    assert aten_fast.fast_aten_mean(_fake((4, 8), torch.int64)) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_amax(_fake((4, 8), torch.int16), [1]) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_argmax(_fake((0, 8)), 1) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_argmax(_fake((4, 8)), 2) is aten_fast.NOT_HANDLED
    assert aten_fast.fast_aten_sum(_fake((4, 8)), [0, 0]) is aten_fast.NOT_HANDLED
    assert fake_backend == []


# ---------------------------------------------------------------------------
# on the GPU
# ---------------------------------------------------------------------------
gpu = pytest.mark.gpu


def _close(got, want, rtol=None, atol=None):
    assert isinstance(got, torch_mojo_backend.TorchMojoTensor)
    assert got.device.type == "mojo" and got.dtype == want.dtype and got.shape == want.shape
    torch.testing.assert_close(got.cpu(), want, rtol=rtol, atol=atol)


@gpu
def test_roundtrip_views_and_payload():
    x = torch.randn(4, 6)
    m = x.to("mojo")
    assert isinstance(m, torch_mojo_backend.TorchMojoTensor) and m.device == torch.device("mojo:0")
    assert m._shape == (4, 6) and m._strides == (6, 1) and m._is_contiguous and m._itemsize == 4
    assert m._ptr == m._holder.data_ptr() and m._numel == 24
    assert torch.equal(m.cpu(), x)
    t = m.t()
    assert t._strides == (1, 6) and not t._is_contiguous and t._ptr == m._ptr   # zero-copy view
    assert torch.equal(t.cpu(), x.t())
    assert torch.equal(m.view(2, 12).cpu(), x.view(2, 12))
    assert torch.equal(m[1:3].cpu(), x[1:3])
    assert torch.equal(m.to(torch.bfloat16).cpu(), x.to(torch.bfloat16))


@gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 5e-2)])
def test_eager_gemm_family(dtype, tol):
    a, b, bias = torch.randn(33, 64).to(dtype), torch.randn(64, 48).to(dtype), torch.randn(48).to(dtype)
    am, bm, cm = a.to("mojo"), b.to("mojo"), bias.to("mojo")
    before = aten_fast.fast_aten_addmm.call_count
    _close(torch.addmm(cm, am, bm), torch.addmm(bias, a, b), rtol=tol, atol=tol)
    assert aten_fast.fast_aten_addmm.call_count == before + 1
    _close(torch.mm(am, bm), torch.mm(a, b), rtol=tol, atol=tol)
    w = torch.randn(48, 64).to(dtype)
    x3 = torch.randn(2, 5, 64).to(dtype)
    _close(torch.nn.functional.linear(x3.to("mojo"), w.to("mojo"), cm),
           torch.nn.functional.linear(x3, w, bias), rtol=tol, atol=tol)
    a3, b3 = torch.randn(3, 9, 16).to(dtype), torch.randn(3, 16, 11).to(dtype)
    _close(torch.bmm(a3.to("mojo"), b3.to("mojo")), torch.bmm(a3, b3), rtol=tol, atol=tol)
    with pytest.raises(NotImplementedError, match="aten::addmm is not supported by mojo eager"):
        torch.addmm(cm, am, bm, beta=0.5)


@gpu
def test_eager_softmax_layer_norm_reductions():
    x = torch.randn(6, 10, 12)
    m = x.to("mojo")
    for dim in (0, 1, 2, -1):
        _close(torch.softmax(m, dim), torch.softmax(x, dim), rtol=1e-5, atol=1e-6)
        _close(torch.log_softmax(m, dim), torch.log_softmax(x, dim), rtol=1e-5, atol=1e-5)
    w, b = torch.randn(12), torch.randn(12)
    got = torch.native_layer_norm(m, [12], w.to("mojo"), b.to("mojo"), 1e-5)
    want = torch.native_layer_norm(x, [12], w, b, 1e-5)
    for g, t, tol in zip(got, want, (1e-5, 1e-5, 1e-4)):
        _close(g, t, rtol=tol, atol=tol)
    assert got[1].shape == (6, 10, 1) and got[1].dtype == torch.float32
    _close(torch.nn.functional.layer_norm(m, [12]), torch.nn.functional.layer_norm(x, [12]),
           rtol=1e-5, atol=1e-5)
    _close(m.sum(), x.sum(), rtol=1e-5, atol=1e-4)
    _close(m.sum(dim=1), x.sum(dim=1), rtol=1e-5, atol=1e-5)
    _close(m.mean(dim=(0, 2), keepdim=True), x.mean(dim=(0, 2), keepdim=True), rtol=1e-5, atol=1e-6)
    _close(m.mean(), x.mean(), rtol=1e-5, atol=1e-6)
    _close(torch.amax(m, dim=-1), torch.amax(x, dim=-1), rtol=0, atol=0)
    _close(torch.argmax(m, dim=1), torch.argmax(x, dim=1), rtol=0, atol=0)
    _close(torch.argmax(m), torch.argmax(x), rtol=0, atol=0)
    ints = torch.randint(-5, 5, (7, 9), dtype=torch.int32)
    _close(ints.to("mojo").sum(dim=1), ints.sum(dim=1), rtol=0, atol=0)
    _close(torch.nn.functional.gelu(m, approximate="tanh"),
           torch.nn.functional.gelu(x, approximate="tanh"), rtol=1e-5, atol=1e-6)


@gpu
def test_eager_argmax_vocab_planted_max():
    x = torch.randn(256, 50257)
    planted = torch.randint(0, 50257, (256,))
    x[torch.arange(256), planted] = 100.0
    assert torch.equal(torch.argmax(x.to("mojo"), dim=-1).cpu(), planted)


@gpu
def test_eager_sdpa_decode_step_takes_the_decode_kernel(monkeypatch):
    """One query per head, no mask: the eager twin must launch the memory-bound decode kernel, not
    the 128-query MFMA kernel that also accepts the shapes."""
    hip_ops = aten_fast.hip_ops
    decode_calls, fused_calls = [], []
    real_decode, real_fused = hip_ops.attention_decode, hip_ops.attention
    monkeypatch.setattr(hip_ops, "attention_decode",
                        lambda *a, **kw: decode_calls.append(1) or real_decode(*a, **kw))
    monkeypatch.setattr(hip_ops, "attention", lambda *a, **kw: fused_calls.append(1) or real_fused(*a, **kw))
    g = torch.Generator().manual_seed(0)
    q = torch.randn(3, 12, 1, 64, generator=g).bfloat16()
    k = torch.randn(3, 12, 208, 64, generator=g).bfloat16()
    v = torch.randn(3, 12, 208, 64, generator=g).bfloat16()
    got = torch.nn.functional.scaled_dot_product_attention(q.to("mojo"), k.to("mojo"), v.to("mojo"))
    assert len(decode_calls) == 1 and not fused_calls
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    _close(got.float(), want, rtol=2e-2, atol=2e-2)


@gpu
def test_out_variants_follow_the_dtype_policy():
    """out= overloads (reference mojo_device_aten_ops.py:155-207, aten::mean.out :761): compute,
    then a strided, casting copy into out; safe_cast / exact policies; wrong device or shape."""
    x = torch.randn(6, 10)
    m = x.to("mojo")
    out = torch.empty(6, device="mojo")
    ret = torch.mean(m, dim=1, out=out)
    assert ret is out
    torch.testing.assert_close(out.cpu(), x.mean(dim=1), rtol=1e-5, atol=1e-6)
    # safe_cast: a float32 mean may land in a float64 destination, not in an integer one
    wide = torch.empty(6, dtype=torch.float64, device="mojo")
    torch.mean(m, dim=1, out=wide)
    torch.testing.assert_close(wide.cpu(), x.double().mean(dim=1), rtol=1e-5, atol=1e-6)
    with pytest.raises(RuntimeError, match="can't be cast"):
        torch.mean(m, dim=1, out=torch.empty(6, dtype=torch.int32, device="mojo"))
    # a strided destination: every other column of a wider buffer
    buf = torch.zeros(6, 2, device="mojo")
    torch.sum(m, dim=[1], out=buf[:, 1])
    got = buf.cpu()
    torch.testing.assert_close(got[:, 1], x.sum(dim=1), rtol=1e-5, atol=1e-5)
    assert bool((got[:, 0] == 0).all())
    # exact policy
    a, b = torch.randn(5, 7), torch.randn(7, 3)
    dst = torch.empty(5, 3, device="mojo")
    assert torch.mm(a.to("mojo"), b.to("mojo"), out=dst) is dst
    torch.testing.assert_close(dst.cpu(), a @ b, rtol=1e-4, atol=1e-4)
    with pytest.raises(RuntimeError, match="can't be cast"):
        torch.mm(a.to("mojo"), b.to("mojo"), out=torch.empty(5, 3, dtype=torch.float64, device="mojo"))
    idx = torch.empty(6, dtype=torch.int64, device="mojo")
    torch.argmax(m, dim=1, out=idx)
    assert torch.equal(idx.cpu(), x.argmax(dim=1))
    with pytest.raises(RuntimeError, match="shape"):
        torch.mean(m, dim=1, out=torch.empty(5, device="mojo"))
    with pytest.raises((RuntimeError, TypeError)):
        torch.mean(m, dim=1, out=torch.empty(6))             # a host destination


@gpu
def test_mojo_backend_over_mojo_tensors_returns_zero_copy_wrappers():
    """torch.compile(backend=mojo_backend) over eager mojo tensors (reference
    torch_compile_backend/compiler.py:496-532, tests/test_compile_mojo_device.py): inputs are
    consumed in place, results are mojo tensors."""
    from torch_mojo_backend import mojo_backend

    def fn(x, w, b):
        h = torch.nn.functional.linear(x, w, b)
        return torch.softmax(h, dim=-1), h.sum(dim=0), None

    x, w, b = torch.randn(9, 16), torch.randn(12, 16), torch.randn(12)
    xm, wm, bm = x.to("mojo"), w.to("mojo"), b.to("mojo")
    probs, sums, nothing = torch.compile(fn, backend=mojo_backend, fullgraph=True)(xm, wm, bm)
    assert nothing is None
    want = fn(x, w, b)
    _close(probs, want[0], rtol=1e-4, atol=1e-5)
    _close(sums, want[1], rtol=1e-4, atol=1e-4)
    # a non-contiguous input view and an output that is a view of an input
    def fn2(x):
        return x + 1.0, x.t()

    y, xt = torch.compile(fn2, backend=mojo_backend, fullgraph=True)(xm.t())
    _close(y, x.t() + 1.0, rtol=0, atol=0)
    _close(xt, x, rtol=0, atol=0)
    assert xt._ptr == xm._ptr                                  # adopted, not copied


@gpu
def test_mojo_backend_over_host_tensors_copies_in_and_out(monkeypatch):
    """The workload's CPU-resident configuration: a float32 GPT-2-shaped module that lives on the
    host, compiled with mojo_backend. There is no CPU kernel path: parameters and inputs cross to
    the HIP device at every call, results come back as host tensors. Every kind of write to a
    host parameter is seen by the next call, as with the reference's aliasing import of host
    buffers (torch_compile_backend/compiler.py:535-566): in place, through `.data`, through the
    numpy view. The fused attention step still runs (the causal verdict is taken on the host
    buffer while the graph is built and travels with each device copy)."""
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.torch_compile_backend import compiler

    monkeypatch.delenv("TORCH_MOJO_BACKEND_CACHE_HOST_PARAMETERS", raising=False)
    model = build_gpt2_small(seed=0, n_layer=2)
    idx = seeded_tokens(1, 128, seed=0)
    fused = []
    real = compiler.aten_functions.hip_ops.softmax_scaled
    monkeypatch.setattr(compiler.aten_functions.hip_ops, "softmax_scaled",
                        lambda *a, **kw: (fused.append(1), real(*a, **kw))[1])
    with torch.no_grad():
        want_logits, want_next = model(idx)
        compiled = torch.compile(model, backend=mojo_backend, fullgraph=True)
        made = compiler._DEVICE_COPIES["made"]
        logits, nxt = compiled(idx)
        logits2, _ = compiled(idx)
    assert logits.device.type == "cpu" and nxt.device.type == "cpu"
    torch.testing.assert_close(logits, want_logits, rtol=1e-4, atol=1e-4)
    assert torch.equal(nxt, torch.argmax(logits[:, -1, :], dim=-1))
    assert compiler._DEVICE_COPIES["made"] == made                    # nothing is kept
    assert torch.equal(logits, logits2)
    assert len(fused) == 4                                            # two layers, two calls
    with torch.no_grad():
        model.transformer.ln_f.bias.add_(1.0)                         # bumps the version counter
        logits3, _ = compiled(idx)
        want3, _ = model(idx)
        torch.testing.assert_close(logits3, want3, rtol=1e-4, atol=1e-4)
        model.transformer.h[0].mlp.c_fc.weight.data.mul_(0.5)         # does not
        logits4, _ = compiled(idx)
        want4, _ = model(idx)
        assert not torch.allclose(want4, want3, atol=1e-3)
        torch.testing.assert_close(logits4, want4, rtol=1e-4, atol=1e-4)
        model.transformer.ln_f.weight.detach().numpy()[:] *= 2.0      # nor does numpy
        logits5, _ = compiled(idx)
        want5, _ = model(idx)
        torch.testing.assert_close(logits5, want5, rtol=1e-4, atol=1e-4)


@gpu
def test_kept_parameter_copies_are_opt_in_and_can_be_dropped(monkeypatch):
    """TORCH_MOJO_BACKEND_CACHE_HOST_PARAMETERS=1: parameters cross once and are reused while
    data pointer and version counter stand; a write the counter misses needs
    `invalidate_device_copies`."""
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.torch_compile_backend import compiler

    monkeypatch.setenv("TORCH_MOJO_BACKEND_CACHE_HOST_PARAMETERS", "1")
    model = build_gpt2_small(seed=0, n_layer=1)
    idx = seeded_tokens(1, 64, seed=0)
    with torch.no_grad():
        compiled = torch.compile(model, backend=mojo_backend, fullgraph=True)
        before = dict(compiler._DEVICE_COPIES)
        compiled(idx)
        made = compiler._DEVICE_COPIES["made"] - before["made"]
        compiled(idx)
        assert made > 0 and compiler._DEVICE_COPIES["made"] - before["made"] == made
        assert compiler._DEVICE_COPIES["reused"] - before["reused"] >= made
        model.transformer.ln_f.bias.add_(1.0)                         # seen: the counter moved
        got, _ = compiled(idx)
        want, _ = model(idx)
        torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)
        model.transformer.ln_f.weight.data.mul_(2.0)                  # not seen ...
        stale, _ = compiled(idx)
        want, _ = model(idx)
        assert not torch.allclose(stale, want, atol=1e-3)
        assert compiler.invalidate_device_copies(model) >= made       # ... until dropped
        got, _ = compiled(idx)
        torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)


def test_out_of_memory_launch_status_becomes_torch_out_of_memory_error(monkeypatch):
    """Host-only: a launcher that reports hipErrorOutOfMemory (status 2) surfaces as
    torch.OutOfMemoryError, any other failure as HipKernelError naming the op (the reference maps
    its kernels' OOM markers the same way, aten_fast.py:730-751, tests/test_tensor_spec_oom.py)."""
    from torch_mojo_backend.eager_kernels import hip_ops

    with pytest.raises(torch.OutOfMemoryError, match="tmb_gemm"):
        hip_ops._check("tmb_gemm", 2)
    with pytest.raises(hip_ops.HipKernelError, match="tmb_softmax_rows failed.*invalid argument"):
        hip_ops._check("tmb_softmax_rows", -1)
    assert hip_ops._check("tmb_gemm", 0) is None

    class _Lib:
        def tmb_softmax_rows(self, *a):
            return 2

    class _T:
        dtype, device, shape = torch.float32, torch.device("cuda", 0), (2, 4)

    # through a real launcher: everything up to the launch is stubbed, the status is real
    monkeypatch.setattr(hip_ops, "require_hip", lambda *t: torch.device("cuda", 0))
    monkeypatch.setattr(hip_ops._ek, "lib", lambda: _Lib())
    monkeypatch.setattr(hip_ops, "_stream", lambda: 0)
    monkeypatch.setattr(hip_ops.torch, "empty", lambda *a, **k: torch.zeros(2, 4))
    x = torch.zeros(2, 4)
    with pytest.raises(torch.OutOfMemoryError, match="tmb_softmax_rows"):
        hip_ops.softmax(x, -1)

