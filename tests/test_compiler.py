"""Host logic of the graph surface, runnable without a GPU: registry semantics, error text,
decomposition skipping, the step program (fusion, liveness, output blueprint).

Where a graph has to *execute* on this GPU-less host the hot entries of the registry are
monkeypatched with PyTorch CPU functions — the reference's own "fake backend" pattern
(tests/test_tensor_spec_oom.py:14-143) — so the executor is exercised, not the kernels."""

import operator

import pytest
import torch

import torch_mojo_backend
from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO, MojoCompilerError, mojo_backend
from torch_mojo_backend import aten_functions as af
from torch_mojo_backend.torch_compile_backend import compiler

aten = torch.ops.aten


def test_public_names():
    for name in ("mojo_backend", "MAPPING_TORCH_ATEN_TO_MOJO", "MojoCompilerError",
                 "get_accelerators"):
        assert hasattr(torch_mojo_backend, name)
    assert torch_mojo_backend.get_accelerators()[-1] == torch.device("cpu")


def test_registry_has_the_hot_entries_and_identity_functions():
    for op in (aten.mm, aten.addmm, aten.bmm, aten.linear, aten._softmax, aten.softmax,
               aten._log_softmax, aten.native_layer_norm, aten.sum, aten.mean, aten.amax,
               aten.argmax, aten.gelu):
        assert op in MAPPING_TORCH_ATEN_TO_MOJO
        assert hasattr(MAPPING_TORCH_ATEN_TO_MOJO[op], "call_count")
    for fn in (operator.add, operator.getitem, max, min, str):
        assert MAPPING_TORCH_ATEN_TO_MOJO[fn] is fn
    assert MAPPING_TORCH_ATEN_TO_MOJO is compiler.MAPPING_TORCH_ATEN_TO_MOJO is af.MAPPING_TORCH_ATEN_TO_MOJO


def test_map_to_removes_decompositions_and_rejects_other_keys():
    assert len(af.DECOMPOSITION_TABLE) < af.original_decomposition_table_size
    for overload in (aten.addmm.default, aten.native_layer_norm.default, aten._softmax.default,
                     aten._log_softmax.default, aten.gelu.default, aten.mean.dim):
        assert overload not in af.DECOMPOSITION_TABLE
    with pytest.raises(TypeError, match="OpOverload"):
        af.map_to("aten.tanh")(lambda x: x)
    # decorator registers, counts and pops a single overload
    table_had = aten.hardswish.default in af.DECOMPOSITION_TABLE
    saved = af.DECOMPOSITION_TABLE.get(aten.hardswish.default)
    try:
        @af.map_to(aten.hardswish.default)
        def my_hardswish(x):
            return torch.nn.functional.hardswish(x)

        assert MAPPING_TORCH_ATEN_TO_MOJO[aten.hardswish.default] is my_hardswish
        assert aten.hardswish.default not in af.DECOMPOSITION_TABLE
        my_hardswish(torch.zeros(2))
        assert my_hardswish.call_count == 1
    finally:
        MAPPING_TORCH_ATEN_TO_MOJO.pop(aten.hardswish.default, None)
        if table_had:
            af.DECOMPOSITION_TABLE[aten.hardswish.default] = saved


def test_unmapped_op_raises_with_the_reference_text(monkeypatch):
    monkeypatch.delitem(MAPPING_TORCH_ATEN_TO_MOJO, aten.cos)

    def fn(x):
        return torch.cos(x) + 1

    with pytest.raises(Exception) as info:
        torch.compile(fn, backend=mojo_backend)(torch.randn(3))
    text = str(info.value)
    assert "The aten function is not supported by the Mojo backend yet" in text
    assert "torch._ops.aten.aten::cos" in text or "cos" in text
    assert "Failing at node" in text
    assert "https://github.com/gabrieldemarmiesse/torch-mojo-backend/issues" in text
    assert "MAPPING_TORCH_ATEN_TO_MOJO" in text
    assert "return torch.cos(x) + 1" in text   # the user stack trace


def test_exception_in_mapping_function_is_wrapped(monkeypatch):
    def broken(x):
        raise ValueError("boom from mapping")

    monkeypatch.setitem(MAPPING_TORCH_ATEN_TO_MOJO, aten.cos, broken)
    with pytest.raises(Exception) as info:
        torch.compile(lambda x: torch.cos(x), backend=mojo_backend)(torch.randn(3))
    text = str(info.value)
    assert "boom from mapping" in text and "There was an error when executing the function" in text
    cause = info.value
    while cause is not None and not isinstance(cause, MojoCompilerError):
        cause = cause.__cause__ or cause.__context__
    assert isinstance(cause, MojoCompilerError)


def test_user_can_override_an_entry(monkeypatch):
    calls = []

    def my_tanh(x):
        calls.append(1)
        return torch.tanh(x) * 0 + 7

    monkeypatch.setitem(MAPPING_TORCH_ATEN_TO_MOJO, aten.tanh, my_tanh)
    out = torch.compile(lambda x: torch.tanh(x), backend=mojo_backend)(torch.randn(4))
    assert calls and torch.equal(out, torch.full((4,), 7.0))


@pytest.fixture()
def cpu_hot_ops(monkeypatch):
    """Stand-ins so graphs can execute on this host; they record what the executor asked for."""
    log = []

    def rec(name, fn):
        def run(*a, **k):
            log.append(name)
            return fn(*a, **k)
        run.__name__ = name
        return run

    fake = {
        aten.addmm: rec("addmm", lambda i, a, b, **k: torch.addmm(i, a, b, **k)),
        aten.mm: rec("mm", torch.mm),
        aten.bmm: rec("bmm", torch.bmm),
        aten._softmax: rec("_softmax", lambda x, d, h: torch.softmax(x, d)),
        aten.gelu: rec("gelu", lambda x, approximate="none": torch.nn.functional.gelu(x, approximate=approximate)),
        aten.argmax: rec("argmax", torch.argmax),
    }

    def ln(x, shape, w, b, eps):
        log.append("ln_first_only" if af._only_first_output_used() else "ln_all")
        return torch.native_layer_norm(x, shape, w, b, eps)

    fake[aten.native_layer_norm] = ln
    for k, v in fake.items():
        monkeypatch.setitem(MAPPING_TORCH_ATEN_TO_MOJO, k, v)
    # the fusion pass keys on the built-in entries; point it at the stand-ins
    monkeypatch.setattr(compiler, "_BUILTIN_ADDMM", fake[aten.addmm])
    monkeypatch.setattr(compiler, "_BUILTIN_GELU", fake[aten.gelu])
    monkeypatch.setattr(compiler, "_BUILTIN_LAYER_NORM", ln)
    # these graphs stay on the host with the stand-ins, also where a HIP device exists
    monkeypatch.setattr(compiler, "_hip_available", lambda: False)
    monkeypatch.setattr(af, "addmm_gelu",
                        rec("addmm_gelu", lambda i, a, b, approx, twice=False: torch.nn.functional.gelu(
                            torch.addmm(i, a, b), approximate=approx)))
    return log


def test_executor_runs_a_model_and_fuses_bias_gelu(cpu_hot_ops):
    torch.manual_seed(0)
    mlp = torch.nn.Sequential(torch.nn.LayerNorm(16), torch.nn.Linear(16, 32),
                              torch.nn.GELU(approximate="tanh"), torch.nn.Linear(32, 8)).eval()
    x = torch.randn(2, 5, 16)
    with torch.no_grad():
        want = mlp(x)
        got = torch.compile(mlp, backend=mojo_backend, fullgraph=True)(x)
    torch.testing.assert_close(got, want)
    assert "addmm_gelu" in cpu_hot_ops and "gelu" not in cpu_hot_ops
    assert cpu_hot_ops.count("addmm") == 1          # the second Linear
    assert "ln_first_only" in cpu_hot_ops           # inference graph: statistics are dead


class _TwoBlocks(torch.nn.Module):
    """x <- x + proj(norm(x)), twice, then a final norm: the residual stream of a decoder."""

    def __init__(self):
        super().__init__()
        self.n1, self.n2, self.nf = (torch.nn.LayerNorm(16) for _ in range(3))
        self.p1, self.p2 = torch.nn.Linear(16, 16), torch.nn.Linear(16, 16)
        self.head = torch.nn.Linear(16, 4, bias=False)

    def forward(self, x):
        x = x + self.p1(self.n1(x))
        x = x + self.p2(self.n2(x))
        return self.head(self.nf(x))


def _plans_of(model, x, monkeypatch):
    seen = []
    real = compiler._GraphFactory._widen_residual_stream

    def spy(plans):
        real(plans)
        seen.append({n.name: p for n, p in plans.items() if p is not None})

    monkeypatch.setattr(compiler._GraphFactory, "_widen_residual_stream", staticmethod(spy))
    with torch.no_grad():
        out = torch.compile(model, backend=mojo_backend, fullgraph=True)(x)
    return out, (seen[-1] if seen else {})


def test_residual_stream_of_a_16_bit_graph_is_kept_in_float32(cpu_hot_ops, monkeypatch):
    torch.manual_seed(0)
    model = _TwoBlocks().eval().to(torch.bfloat16)
    x = torch.randn(2, 5, 16).to(torch.bfloat16)
    import copy
    with torch.no_grad():    # before compiling: dynamo's guards hold weak references to the
        want = copy.deepcopy(model).float()(x.float())   # parameters, which .float() cannot swap
    out, plans = _plans_of(model, x, monkeypatch)
    residual = [p for p in plans.values() if p[0] == "residual"]
    norms = [p for p in plans.values() if p[0] == "wide_ln"]
    # both residual adds hand float32 on (their consumers are the next add and layer norms);
    # the two layer norms behind them read float32 and produce bfloat16
    assert len(residual) == 2 and all(p[6] is torch.float32 for p in residual)
    assert len(norms) == 2 and all(p[1] is torch.bfloat16 for p in norms)
    assert out.dtype == torch.bfloat16
    torch.testing.assert_close(out.float(), want, rtol=5e-2, atol=5e-2)


def test_residual_stream_stays_narrow_when_something_else_reads_it(cpu_hot_ops, monkeypatch):
    class Leaky(_TwoBlocks):
        def forward(self, x):
            x = x + self.p1(self.n1(x))
            y = x + self.p2(self.n2(x))
            return self.head(self.nf(y)), x          # the first stream value is a graph output

    torch.manual_seed(0)
    model = Leaky().eval().to(torch.bfloat16)
    (out, leaked), plans = _plans_of(model, torch.randn(2, 5, 16).to(torch.bfloat16), monkeypatch)
    residual = [p for p in plans.values() if p[0] == "residual"]
    assert sorted(str(p[6]) for p in residual) == ["None", "torch.float32"]
    assert leaked.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
    # float32 graphs and the bit-identical mode leave the graph's dtypes alone
    _, plans32 = _plans_of(_TwoBlocks().eval(), torch.randn(2, 5, 16), monkeypatch)
    assert all(p[6] is None for p in plans32.values() if p[0] == "residual")
    monkeypatch.setenv("TORCH_MOJO_BACKEND_ROUND_LIKE_UNFUSED", "1")
    torch.compiler.reset()
    _, plans_twice = _plans_of(_TwoBlocks().eval().to(torch.bfloat16),
                               torch.randn(2, 5, 16).to(torch.bfloat16), monkeypatch)
    assert plans_twice == {}                          # the widening pass is not even entered


def test_fusion_can_be_switched_off(cpu_hot_ops, monkeypatch):
    monkeypatch.setenv("TORCH_MOJO_BACKEND_NO_FUSION", "1")
    lin = torch.nn.Sequential(torch.nn.Linear(8, 8), torch.nn.GELU()).eval()
    x = torch.randn(3, 8)
    with torch.no_grad():
        torch.testing.assert_close(torch.compile(lin, backend=mojo_backend)(x), lin(x))
    assert "gelu" in cpu_hot_ops and "addmm_gelu" not in cpu_hot_ops


def test_layer_norm_statistics_kept_when_used(cpu_hot_ops):
    def fn(x, w, b):
        out, mean, rstd = torch.native_layer_norm(x, [8], w, b, 1e-5)
        return out, mean, rstd

    x, w, b = torch.randn(4, 8), torch.randn(8), torch.randn(8)
    got = torch.compile(fn, backend=mojo_backend)(x, w, b)
    want = fn(x, w, b)
    for g, t in zip(got, want):
        torch.testing.assert_close(g, t)
    assert "ln_all" in cpu_hot_ops


def test_outputs_none_ints_and_dynamic_shapes(cpu_hot_ops):
    def fn(x):
        return x.shape[0] * 2, None, x + 1

    compiled = torch.compile(fn, backend=mojo_backend, dynamic=True)
    for n in (3, 5, 9):
        size, nothing, y = compiled(torch.zeros(n, 2))
        assert size == 2 * n and nothing is None and y.shape == (n, 2) and bool((y == 1).all())


def test_intermediates_are_released_after_their_last_use():
    gm = torch.fx.symbolic_trace(lambda x: torch.ops.aten.add.Tensor(
        torch.ops.aten.mul.Tensor(x, 2), torch.ops.aten.mul.Tensor(x, 3)))
    program = compiler._GraphFactory().create_graph(gm.graph)
    released = [slot for step in program.steps for slot in step.release]
    # both products and the input are dropped once the add has run; the result is kept
    assert sorted(released) == [0, 1, 2]
    assert program.steps[-1].out not in released


def test_padded_copies_are_shared_only_inside_a_graph_run(monkeypatch):
    """The padded copy of a large operand is kept for the next product only while the run-scoped
    dictionary exists: same memory, shape, strides and width give the same copy; anything else,
    and every call outside a run, makes a new one."""
    from torch_mojo_backend.eager_kernels import hip_ops

    monkeypatch.setattr(hip_ops, "_PAD_REUSE_MIN_BYTES", 1 << 10)
    x = torch.randn(64, 33)
    a, b = hip_ops._pad_last(x, 40), hip_ops._pad_last(x, 40)
    assert a is not b and torch.equal(a, b) and a.shape == (64, 40)
    assert torch.equal(a[:, :33], x) and bool((a[:, 33:] == 0).all())
    before = hip_ops.pad_reuse_begin()
    assert before is None
    try:
        a = hip_ops._pad_last(x, 40)
        assert hip_ops._pad_last(x.t().t(), 40) is a          # another view of the same rows
        assert hip_ops._pad_last(x[:32], 40) is not a         # other shape
        assert hip_ops._pad_last(x, 40) is not a              # one entry: the narrower view replaced it
        c = hip_ops._pad_last(x, 48)
        assert c.shape == (64, 48) and hip_ops._pad_last(x, 48) is c
        small = torch.randn(4, 33)
        assert hip_ops._pad_last(small, 40) is not hip_ops._pad_last(small, 40)
        (kept_source, kept_copy), = hip_ops.pad_reuse_active().values()
        assert kept_source is x and kept_copy is c
    finally:
        hip_ops.pad_reuse_end(before)
    assert hip_ops.pad_reuse_active() is None


def test_graph_runs_share_padded_copies_unless_a_node_writes_in_place(cpu_hot_ops):
    from torch.fx.experimental.proxy_tensor import make_fx
    from torch_mojo_backend.eager_kernels import hip_ops

    seen = []

    def spy(a, b):
        seen.append(hip_ops.pad_reuse_active())
        return torch.mm(a, b)

    MAPPING_TORCH_ATEN_TO_MOJO[aten.mm] = spy  # (the fixture restores the entry)
    x, w = torch.randn(4, 6), torch.randn(6, 6)
    pure = make_fx(lambda x, w: torch.mm(torch.mm(x, w), w))(x, w)
    run = compiler.BaseMaxCompiler(pure, [x, w])
    assert run.pad_reuse_module is hip_ops
    out, = run(x, w)
    assert torch.allclose(out, x @ w @ w)
    assert seen == [{}, {}] and seen[0] is seen[1] and hip_ops.pad_reuse_active() is None
    one = make_fx(lambda x, w: torch.mm(x, w))(x, w)
    assert compiler.BaseMaxCompiler(one, [x, w]).pad_reuse_module is None

    def writes(x, w):
        y = torch.mm(x, w)
        torch.add(y, 1.0, out=y)
        return torch.mm(y, w)

    assert compiler.BaseMaxCompiler(make_fx(writes)(x, w), [x, w]).pad_reuse_module is None


class _Attn(torch.nn.Module):
    """Score pipeline of a decoder block, as demo_scripts/gpt2.py writes it."""

    def __init__(self, block=16, causal=True):
        super().__init__()
        mask = torch.tril(torch.ones(block, block)) if causal else (torch.rand(block, block) > 0.3).float()
        mask[:, 0] = 1.0  # no fully masked row
        self.register_buffer("bias", mask.view(1, 1, block, block), persistent=False)

    def forward(self, q, k):
        t = q.shape[-2]
        att = (q @ k.transpose(-2, -1)) * 0.25
        att = att.masked_fill(self.bias[:, :, :t, :t] == 0, float("-inf"))
        return torch.softmax(att, dim=-1)


def test_masked_softmax_rewrite_plans_one_fused_step(cpu_hot_ops, monkeypatch):
    monkeypatch.setattr(compiler, "_BUILTIN_SOFTMAX", MAPPING_TORCH_ATEN_TO_MOJO[aten._softmax])
    programs = []
    real = compiler._GraphFactory.create_graph

    def spy(self, graph):
        programs.append(real(self, graph))
        return programs[-1]

    monkeypatch.setattr(compiler._GraphFactory, "create_graph", spy)
    model = _Attn().eval()
    q, k = torch.randn(2, 3, 8, 4), torch.randn(2, 3, 8, 4)
    with torch.no_grad():
        want = model(q, k)
        got = torch.compile(model, backend=mojo_backend, fullgraph=True)(q, k)
    # host tensors take the unfused branch inside the fused step: same numbers as eager
    torch.testing.assert_close(got, want)
    program = programs[-1]
    names = [compiler._step_name(s) for s in program.steps]
    assert names.count("aten.mul+masked_fill+_softmax (fused)") == 1
    fused = next(s for s in program.steps if s.fn is compiler._FUSED_MASKED_SOFTMAX)
    # the nodes whose work the fused step does are not in the program at all
    remaining = {str(s.node.target) for s in program.steps}
    assert not remaining & {"aten.mul.Tensor", "aten.masked_fill.Scalar", "aten.eq.Scalar",
                            "aten.slice.Tensor"}
    assert fused.args[1] == 0.25 and fused.args[3] == ((2, 0, 8, 1), (3, 0, 8, 1))
    # the scores stay alive until the fused step has read them, then go
    scores_slot = fused.args[0].index
    assert scores_slot in fused.release
    for s in program.steps:
        if s is not fused:
            assert scores_slot not in s.release


def test_masked_softmax_rewrite_leaves_other_patterns_alone(cpu_hot_ops, monkeypatch):
    monkeypatch.setattr(compiler, "_BUILTIN_SOFTMAX", MAPPING_TORCH_ATEN_TO_MOJO[aten._softmax])

    def shared_product(q, k, mask):
        att = (q @ k.transpose(-2, -1)) * 0.5
        return torch.softmax(att.masked_fill(mask == 0, float("-inf")), dim=-1), att  # mul has 2 users

    def finite_fill(q, k, mask):
        att = (q @ k.transpose(-2, -1)) * 0.5
        return torch.softmax(att.masked_fill(mask == 0, -1e9), dim=-1)

    q, k = torch.randn(2, 6, 4), torch.randn(2, 6, 4)
    mask = torch.tril(torch.ones(6, 6))
    for fn in (shared_product, finite_fill):
        want = fn(q, k, mask)
        got = torch.compile(fn, backend=mojo_backend, fullgraph=True)(q, k, mask)
        torch.testing.assert_close(got, want)
        torch.compiler.reset()
    assert cpu_hot_ops.count("_softmax") == 2


def test_causal_verdict_is_cached_and_follows_the_buffer():
    mask = torch.tril(torch.ones(1, 1, 8, 8))
    x = torch.zeros(2, 2, 8, 8)
    # host tensors never qualify (the fused kernel is a device kernel)
    assert compiler._causal_q_len(mask, ((2, 0, 8, 1), (3, 0, 8, 1)), x) == 0


def test_attention_rewrite_plans_one_step_per_block(monkeypatch):
    """The decoder block of demo_scripts/gpt2.py: the whole chain from the q/k/v copies to the
    transposed copy of the context becomes one step that reads q, k, v and the mask buffer."""
    import sys
    sys.path.insert(0, str(__import__("pathlib").Path(__file__).resolve().parents[1] / "torch-max-backend_amd"))
    from demo_scripts.gpt2 import GPT, GPTConfig
    from torch._dynamo.backends.common import aot_autograd
    from functorch.compile import make_boxed_func

    programs = []

    def fw(gm, example_inputs):
        programs.append(compiler._GraphFactory().create_graph(gm.graph))
        return make_boxed_func(gm.forward)

    model = GPT(GPTConfig(block_size=16, vocab_size=50, n_layer=2, n_head=2, n_embd=8)).eval()
    with torch.no_grad():
        torch.compile(model, backend=aot_autograd(fw_compiler=fw, decompositions=af.DECOMPOSITION_TABLE))(
            torch.randint(0, 50, (2, 8)))
    program = programs[-1]
    fused = [s for s in program.steps if s.fn is compiler._FUSED_ATTENTION]
    assert len(fused) == 2
    targets = [str(s.node.target) for s in program.steps]
    assert "aten.bmm.default" not in targets and "aten._softmax.default" not in targets
    assert "aten.clone.default" in targets          # the fused steps sit on the final clones
    assert targets.count("aten.clone.default") == 2
    for s in fused:
        q, k, v, scale, root, slices = s.args
        assert scale == 0.5 and slices == ((2, 0, 8, 1), (3, 0, 8, 1))
        assert len({q.index, k.index, v.index, root.index}) == 4
    monkeypatch.setenv("TORCH_MOJO_BACKEND_NO_ATTENTION_FUSION", "1")
    torch.compiler.reset()
    with torch.no_grad():
        torch.compile(model, backend=aot_autograd(fw_compiler=fw, decompositions=af.DECOMPOSITION_TABLE))(
            torch.randint(0, 50, (2, 8)))
    names = [compiler._step_name(s) for s in programs[-1].steps]
    assert names.count("aten.mul+masked_fill+_softmax (fused)") == 2
    assert not any(s.fn is compiler._FUSED_ATTENTION for s in programs[-1].steps)


def test_residual_add_rewrite(cpu_hot_ops):
    """x + proj(h): addmm -> view -> add becomes one step over (bias, h, w^T, x)."""
    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.proj = torch.nn.Linear(16, 16)

        def forward(self, x, h):
            return x + self.proj(h), torch.tanh(self.proj(h))   # the second use stays a plain addmm

    programs = []
    real = compiler._GraphFactory.create_graph

    def spy(self, graph):
        programs.append(real(self, graph))
        return programs[-1]

    import pytest as _pytest
    mp = _pytest.MonkeyPatch()
    mp.setattr(compiler._GraphFactory, "create_graph", spy)
    try:
        block = Block().eval()
        x, h = torch.randn(2, 5, 16), torch.randn(2, 5, 16)
        with torch.no_grad():
            want = block(x, h)
            got = torch.compile(block, backend=mojo_backend, fullgraph=True)(x, h)
    finally:
        mp.undo()
    torch.testing.assert_close(got[0], want[0])
    torch.testing.assert_close(got[1], want[1])
    names = [compiler._step_name(s) for s in programs[-1].steps]
    assert names.count("aten.addmm+add (fused)") == 1
    fused = next(s for s in programs[-1].steps if s.fn is compiler._FUSED_ADDMM_RESIDUAL)
    assert fused.args[4] == (2, 5, 16)
    assert cpu_hot_ops.count("addmm") == 2     # one inside the fused step's host branch, one plain


def _partitioned_training_graphs(model, idx, targets, partition_fn):
    """Runs one training step through aot_autograd with PyTorch's own kernels and the given
    partitioner; returns ([forward graph, backward graph], parameter gradients)."""
    import torch.nn.functional as F
    from functorch.compile import make_boxed_func
    from torch._dynamo.backends.common import aot_autograd

    graphs = []

    def keep(gm, example_inputs):
        graphs.append(gm)
        return make_boxed_func(gm.forward)

    backend = aot_autograd(fw_compiler=keep, partition_fn=partition_fn,
                           decompositions=af.DECOMPOSITION_TABLE)
    logits, _ = torch.compile(model, backend=backend)(idx)
    F.cross_entropy(logits.view(-1, logits.shape[-1]), targets.view(-1)).backward()
    return graphs, [p.grad.clone() for p in model.parameters()]


def _host_attention_pieces(monkeypatch):
    """The op-by-op route of the two fused training steps, on PyTorch's own CPU kernels."""
    from torch_mojo_backend.eager_kernels import hip_ops

    monkeypatch.setattr(compiler, "_attention_fused_ok", lambda *a: False)
    # (the matchers key on the registry entries being the built-in ones: replace both sides)
    softmax = lambda x, d, h: torch.softmax(x, d)  # noqa: E731
    for op, name, fn in ((aten.bmm, "_BUILTIN_BMM", torch.bmm), (aten._softmax, "_BUILTIN_SOFTMAX", softmax)):
        monkeypatch.setitem(MAPPING_TORCH_ATEN_TO_MOJO, op, fn)
        monkeypatch.setattr(compiler, name, fn)
    monkeypatch.setattr(compiler, "_causal_q_len", lambda *a: -1)
    monkeypatch.setattr(hip_ops, "softmax_backward",
                        lambda g, o, d, log: aten._softmax_backward_data(g, o, d, o.dtype))


def test_training_partition_replaces_attention_forward_and_backward(monkeypatch):
    """A 16-bit attention chain and its backward nodes become the two fused steps: the forward
    graph hands over q, k, v, the output and the log-sum-exp, nothing of size [tokens, tokens]
    exists in either graph, and (on the op-by-op route, which runs on this host) the gradients are
    those of PyTorch's own split."""
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch._functorch.partitioners import default_partition

    _host_attention_pieces(monkeypatch)
    idx, targets = seeded_tokens(2, 8, seed=0), seeded_tokens(2, 8, seed=1)
    make = lambda: build_gpt2_small(seed=0, n_layer=2).bfloat16()  # noqa: E731
    plain, want = _partitioned_training_graphs(make(), idx, targets, default_partition)
    (fw, bw), got = _partitioned_training_graphs(make(), idx, targets,
                                                 compiler.attention_recompute_partition)
    for g, w in zip(got, want):
        scale = w.float().abs().max().item() + 1e-12
        assert (g.float() - w.float()).abs().max().item() <= 3e-2 * scale  # bf16, other op order
    count = lambda gm, target: sum(1 for n in gm.graph.nodes if n.target is target)  # noqa: E731
    assert count(fw, compiler.attention_train_forward) == 2
    assert count(bw, compiler.attention_train_backward) == 2
    for gm in (fw, bw):
        assert count(gm, aten.bmm.default) == 0 and count(gm, aten._softmax.default) == 0
        assert count(gm, aten._softmax_backward_data.default) == 0
        for n in gm.graph.nodes:
            val = n.meta.get("val")
            if isinstance(val, torch.Tensor) and val.dim() >= 3:
                assert tuple(val.shape[-2:]) != (8, 8), n.name
    assert count(plain[1], aten.bmm.default) == 8  # PyTorch's split: four per block
    # the gradient of the packed q/k/v projection comes out of the backward step as one tensor
    assert count(plain[1], aten.cat.default) == 2 and count(bw, aten.cat.default) == 0


def test_training_partition_recomputes_attention_scores_and_forward_fuses(monkeypatch):
    """Where the backward nodes of a chain cannot be replaced, the chain is tagged for
    recomputation instead."""
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch._functorch.partitioners import default_partition

    monkeypatch.setattr(compiler, "_fuse_attention_backward", lambda *a: False)

    idx, targets = seeded_tokens(2, 8, seed=0), seeded_tokens(2, 8, seed=1)
    make = lambda: build_gpt2_small(seed=0, n_layer=2).bfloat16()  # noqa: E731
    plain, want = _partitioned_training_graphs(make(), idx, targets, default_partition)
    graphs, got = _partitioned_training_graphs(make(), idx, targets,
                                               compiler.attention_recompute_partition)
    for g, w in zip(got, want):
        torch.testing.assert_close(g, w, rtol=0, atol=0)  # same ops in the same order
    fw, bw = graphs
    # a float32 graph is split exactly as PyTorch would: the kernel only takes 16-bit heads
    f32, _ = _partitioned_training_graphs(build_gpt2_small(seed=0, n_layer=2), idx, targets,
                                          compiler.attention_recompute_partition)
    assert len([n for n in f32[1].graph.nodes if n.target is aten._softmax.default]) == 0

    def saved_score_matrices(gm):
        outs = gm.graph.output_node().args[0]
        return [o for o in outs if isinstance(o, torch.fx.Node)
                and tuple(o.meta["val"].shape[-2:]) == (8, 8) and o.meta["val"].dim() >= 3
                and o.meta["val"].dtype.is_floating_point]

    # PyTorch's split hands the probabilities to backward; ours hands over none of the
    # [.., tokens, tokens] matrices and the forward graph fuses both attentions
    assert saved_score_matrices(plain[0]) and not saved_score_matrices(fw)
    rewrites = compiler._GraphFactory._fuse_masked_softmax(fw.graph)
    assert len(compiler._GraphFactory._fuse_attention(rewrites)) == 2
    assert len(compiler._GraphFactory._fuse_attention(
        compiler._GraphFactory._fuse_masked_softmax(plain[0].graph))) == 0
    # backward rebuilds the probabilities: one softmax per block, fusable with its mask
    softmaxes = [n for n in bw.graph.nodes if n.target is aten._softmax.default]
    assert len(softmaxes) == 2
    bw_rewrites = compiler._GraphFactory._fuse_masked_softmax(bw.graph)
    assert sum(1 for p in bw_rewrites.values() if p is not None and p[0] == "softmax") == 2


def test_training_partition_packs_gradients_only_for_a_packed_projection(monkeypatch):
    """Separate q, k and v projections: the backward step is still put in, but there is no
    concatenation of its three results to replace, so they come back as three tensors; the
    gradients are those of PyTorch's own split."""
    from demo_scripts.gpt2 import seeded_tokens
    from torch._functorch.partitioners import default_partition

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            torch.manual_seed(0)
            self.emb = torch.nn.Embedding(64, 128)
            self.q, self.k, self.v = (torch.nn.Linear(128, 128) for _ in range(3))
            self.head = torch.nn.Linear(128, 64)
            self.register_buffer("mask", torch.tril(torch.ones(8, 8)).view(1, 1, 8, 8))

        def forward(self, idx):
            x = self.emb(idx)
            b, t, c = x.shape
            q, k, v = (m(x).view(b, t, 2, 64).transpose(1, 2) for m in (self.q, self.k, self.v))
            att = (q @ k.transpose(-2, -1)) * 0.125
            att = torch.softmax(att.masked_fill(self.mask[:, :, :t, :t] == 0, float("-inf")), dim=-1)
            y = (att @ v).transpose(1, 2).contiguous().view(b, t, c)
            return self.head(y), None

    _host_attention_pieces(monkeypatch)
    idx, targets = seeded_tokens(2, 8, seed=0) % 64, seeded_tokens(2, 8, seed=1) % 64
    make = lambda: Block().bfloat16()  # noqa: E731
    _, want = _partitioned_training_graphs(make(), idx, targets, default_partition)
    (fw, bw), got = _partitioned_training_graphs(make(), idx, targets,
                                                 compiler.attention_recompute_partition)
    for g, w in zip(got, want):
        scale = w.float().abs().max().item() + 1e-12
        assert (g.float() - w.float()).abs().max().item() <= 3e-2 * scale
    steps = [n for n in bw.graph.nodes if n.target is compiler.attention_train_backward]
    assert len(steps) == 1 and not isinstance(steps[0].args[-1], str)
    assert {u.args[1] for u in steps[0].users} == {0, 1, 2}


def test_training_partition_leaves_graphs_without_attention_alone():
    from torch._functorch.partitioners import default_partition

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.emb, self.lin = torch.nn.Embedding(8, 8), torch.nn.Linear(8, 8)

        def forward(self, idx):
            return torch.softmax(self.lin(self.emb(idx)), -1), None

    idx, targets = torch.tensor([1, 5, 2, 7]), torch.tensor([0, 3, 3, 6])
    results = []
    for partition in (default_partition, compiler.attention_recompute_partition):
        torch.manual_seed(0)
        results.append(_partitioned_training_graphs(Net(), idx, targets, partition))
    (a_graphs, a), (b_graphs, b) = results
    for g, w in zip(b, a):
        torch.testing.assert_close(g, w)
    for ga, gb in zip(a_graphs, b_graphs):
        assert [n.target for n in ga.graph.nodes] == [n.target for n in gb.graph.nodes]


def test_layer_norm_backward_takes_the_residual_gradient_and_the_bias_sums_along(monkeypatch):
    """A two-block decoder's backward graph: every native_layer_norm_backward whose grad_input
    re-joins the residual stream becomes one step that takes the by-passing gradient along and
    hands the bias gradient of the projection in front of it to the sum node; run with host
    stand-ins for the three ops, the rewritten program returns what the graph itself returns."""
    from demo_scripts.gpt2 import build_gpt2_small, seeded_tokens
    from torch._functorch.partitioners import default_partition

    idx, targets = seeded_tokens(2, 8, seed=0), seeded_tokens(2, 8, seed=1)
    graphs, _ = _partitioned_training_graphs(build_gpt2_small(seed=0, n_layer=2), idx, targets,
                                             default_partition)
    bw = graphs[1]
    plans = compiler._GraphFactory._fuse_norm_backward_add(bw.graph)
    kinds = [p[0] for p in plans.values()]
    # the final norm (bias sums only), two norms per block (an addend each; all but the first
    # block's first norm also feed a projection's bias gradient)
    assert kinds.count("ln_bwd_add") == 5 and kinds.count("take") == 4 and kinds.count("colsum") == 4
    with_addend = [p for p in plans.values() if p[0] == "ln_bwd_add" and p[1] is not None]
    assert len(with_addend) == 4 and sum(1 for p in plans.values() if p[0] == "ln_bwd_add" and p[2]) == 4
    order = {n: i for i, n in enumerate(bw.graph.nodes)}
    for node, plan in plans.items():
        if plan[0] == "ln_bwd_add" and plan[1] is not None:
            assert order[plan[1]] < order[node]       # the addend exists when the step runs
        if plan[0] == "colsum":
            assert tuple(node.meta["val"].shape) == plan[2]
    # somebody else's layer-norm backward: nothing is rewritten
    with monkeypatch.context() as mp:
        mp.setitem(MAPPING_TORCH_ATEN_TO_MOJO, aten.native_layer_norm_backward, lambda *a: None)
        assert compiler._GraphFactory._fuse_norm_backward_add(bw.graph) == {}

    # execute: PyTorch's kernels behind every entry the backward graph uses
    calls = []

    def ln_bwd(*a):
        calls.append("ln_bwd")
        return aten.native_layer_norm_backward.default(*a)

    def add(a, b, alpha=1):
        calls.append("add")
        return torch.add(a, b, alpha=alpha)

    def total(x, dim=None, keepdim=False, dtype=None):
        calls.append("sum")
        return torch.sum(x, dim, keepdim, dtype=dtype) if dim is not None else torch.sum(x, dtype=dtype)

    for op, name, fn in ((aten.native_layer_norm_backward, "_BUILTIN_LAYER_NORM_BACKWARD", ln_bwd),
                         (aten.add, "_BUILTIN_ADD", add), (aten.sum, "_BUILTIN_SUM", total)):
        monkeypatch.setitem(MAPPING_TORCH_ATEN_TO_MOJO, op, fn)
        monkeypatch.setattr(compiler, name, fn)
    for op in {n.target for n in bw.graph.nodes if n.op == "call_function"}:
        key = op if op in MAPPING_TORCH_ATEN_TO_MOJO else getattr(op, "overloadpacket", op)
        if key not in (aten.native_layer_norm_backward, aten.add, aten.sum, operator.getitem):
            monkeypatch.setitem(MAPPING_TORCH_ATEN_TO_MOJO, key, op if key is op else getattr(torch.ops.aten, key.__name__))
    program = compiler._GraphFactory().create_graph(bw.graph)
    fused = [s for s in program.steps if s.fn is compiler._FUSED_NORM_BACKWARD_ADD]
    assert len(fused) == 5
    assert sum(1 for s in program.steps if s.fn is compiler._TAKE_COLUMN_SUMS) == 4
    placeholders = [n for n in bw.graph.nodes if n.op == "placeholder"]
    torch.manual_seed(3)
    inputs = []
    for p in placeholders:
        v = p.meta["val"]
        if v.dtype.is_floating_point:
            inputs.append(torch.randn(v.shape, dtype=v.dtype))
        else:
            inputs.append(torch.randint(0, 2 if v.dtype == torch.bool else 50, tuple(v.shape)).to(v.dtype))
    want = bw(*inputs)
    env = [None] * len(program.slots)
    for slot, value in zip(program.input_slots, inputs):
        env[slot] = value
    for slot, value in program.constants:
        env[slot] = value
    for step in program.steps:
        a = compiler._materialize(step.args, env) if step.dynamic_args else step.args
        k = compiler._materialize(step.kwargs, env) if step.dynamic_kwargs else step.kwargs
        env[step.out] = step.fn(*a, **k)
        for slot in step.release:
            env[slot] = None
    got = compiler._materialize(program.output_template, env)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        if w is None:
            assert g is None
        else:
            torch.testing.assert_close(g, w, rtol=1e-5, atol=1e-6)
    # the four joins ran inside the fused steps' host route, the four bias sums as well
    assert calls.count("ln_bwd") == 5
