"""HIP-graph replays of an inference graph (TORCH_MOJO_BACKEND_HIP_GRAPH=1): every replay is
compared, bit for bit, with the same step program run step by step, with ordinary work and a
synchronisation between the replays."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _model(layers=2):
    from demo_scripts.gpt2 import build_gpt2_small
    return build_gpt2_small(seed=0, n_layer=layers).bfloat16().cuda().eval()


def _both_ways(compiled, idx, monkeypatch):
    """(result with replays allowed, result step by step) of the same compiled module."""
    monkeypatch.setenv("TORCH_MOJO_BACKEND_HIP_GRAPH", "1")
    with torch.no_grad():
        got = compiled(idx)[0]
    monkeypatch.setenv("TORCH_MOJO_BACKEND_HIP_GRAPH", "0")
    with torch.no_grad():
        want = compiled(idx)[0]
    torch.cuda.synchronize()
    return got, want


def test_inference_graph_is_recorded_once_and_every_replay_matches(monkeypatch):
    from demo_scripts.gpt2 import seeded_tokens
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.torch_compile_backend import compiler

    model = _model()
    compiled = torch.compile(model, backend=mojo_backend)
    before = dict(compiler.GRAPH_REPLAYS)
    kept = []
    for seed in range(6):
        idx = seeded_tokens(2, 64, seed=seed).cuda()
        got, want = _both_ways(compiled, idx, monkeypatch)
        assert got.shape == (2, 64, 50257) and torch.equal(got, want), seed
        kept.append((got, want))     # results stay what they were when later replays run
    assert compiler.GRAPH_REPLAYS["recorded"] - before["recorded"] == 1
    assert compiler.GRAPH_REPLAYS["replayed"] - before["replayed"] == 5   # the first call only looks
    for got, want in kept:
        assert torch.equal(got, want)
    # another shape: a graph of its own (dynamo may also hand over a new program)
    idx = seeded_tokens(3, 32, seed=9).cuda()
    for _ in range(3):
        got, want = _both_ways(compiled, idx, monkeypatch)
        assert torch.equal(got, want)


def test_replays_read_the_weights_where_they_are_and_give_way_to_an_edited_buffer(monkeypatch):
    from demo_scripts.gpt2 import seeded_tokens
    from torch_mojo_backend import mojo_backend
    from torch_mojo_backend.torch_compile_backend import compiler

    model = _model(1)
    compiled = torch.compile(model, backend=mojo_backend)
    idx = seeded_tokens(2, 32, seed=1).cuda()
    for _ in range(3):
        first, _ = _both_ways(compiled, idx, monkeypatch)
    replayed = compiler.GRAPH_REPLAYS["replayed"]
    # a weight written in place, also past the version counter: the replay reads the new values
    with torch.no_grad():
        model.transformer.h[0].mlp.c_fc.weight.data.mul_(0.5)
    got, want = _both_ways(compiled, idx, monkeypatch)
    assert compiler.GRAPH_REPLAYS["replayed"] == replayed + 1
    assert torch.equal(got, want) and not torch.equal(got, first)
    # the mask buffer edited in place (what the steps decided from it while the graph was recorded
    # no longer holds): that call runs step by step, and a new graph is recorded afterwards
    bias = model.transformer.h[0].attn.bias
    bias[..., 0, 1] = 1
    replayed = compiler.GRAPH_REPLAYS["replayed"]
    got, want = _both_ways(compiled, idx, monkeypatch)
    assert compiler.GRAPH_REPLAYS["replayed"] == replayed
    assert torch.equal(got, want)
    for _ in range(3):
        got, want = _both_ways(compiled, idx, monkeypatch)
        assert torch.equal(got, want)
    assert compiler.GRAPH_REPLAYS["replayed"] >= replayed + 1
