"""Embedding lookup (``aten.embedding``): the gather kernel through the C ABI, the graph mapping
and the eager ``mojo`` device. A gather moves bits, so every comparison is exact."""

import numpy as np
import pytest
import torch

import oracle
from helpers import seeded


def _ops():
    from torch_mojo_backend.eager_kernels import hip_ops
    return hip_ops


def test_oracle_gather_is_numpy_take_with_clamped_indices():
    rng = np.random.default_rng(3)
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        table = seeded((37, 10), seed=1, dtype=dtype)
        idx = torch.from_numpy(rng.integers(-5, 45, size=(4, 9)))
        want = table[idx.clamp(0, 36)]
        assert torch.equal(oracle.embedding(table, idx), want)
        assert torch.equal(oracle.embedding(table, idx.to(torch.int32)), want)
    # brute force, one element at a time, on a tiny case
    table = torch.arange(12, dtype=torch.float32).reshape(4, 3)
    idx = torch.tensor([3, 0, 0, 2])
    got = oracle.embedding(table, idx)
    for i, r in enumerate(idx.tolist()):
        for c in range(3):
            assert got[i, c].item() == r * 3 + c
    assert oracle.embedding(table, torch.zeros((0, 2), dtype=torch.int64)).shape == (0, 2, 3)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("index_dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("rows_cols", [(50257, 768), (1024, 768), (37, 10), (5, 3), (9, 1), (64, 6)])
def test_gather_matches_the_oracle_bit_for_bit(dtype, index_dtype, rows_cols):
    rows, cols = rows_cols
    table = seeded((rows, cols), seed=11, dtype=dtype)
    g = torch.Generator().manual_seed(12)
    idx = torch.randint(0, rows, (3, 41), generator=g).to(index_dtype)
    got = _ops().embedding(table.cuda(), idx.cuda())
    assert got.dtype == dtype and tuple(got.shape) == (3, 41, cols)
    assert torch.equal(got.cpu(), oracle.embedding(table, idx))
    assert torch.equal(got.cpu(), torch.nn.functional.embedding(idx.long(), table))


@pytest.mark.gpu
def test_gather_edge_cases():
    ops = _ops()
    table = seeded((16, 24), seed=13, dtype=torch.bfloat16).cuda()
    # empty index tensors, scalars and high ranks keep their shape
    assert tuple(ops.embedding(table, torch.zeros((0,), dtype=torch.int64, device="cuda")).shape) == (0, 24)
    assert tuple(ops.embedding(table, torch.tensor(5, device="cuda")).shape) == (24,)
    idx = torch.randint(0, 16, (2, 3, 4, 5), device="cuda")
    assert torch.equal(ops.embedding(table, idx), table[idx])
    # indices outside the table read the nearest valid row, never memory outside it
    wild = torch.tensor([-7, 0, 15, 16, 10 ** 12], device="cuda")
    assert torch.equal(ops.embedding(table, wild), table[wild.clamp(0, 15)])
    # a table that is a strided view, and one whose rows are not 16-byte multiples
    wide = seeded((16, 40), seed=14, dtype=torch.float32).cuda()
    view = wide[:, 3:10]
    assert torch.equal(ops.embedding(view, idx), view[idx])
    # rejected before anything is allocated
    with pytest.raises(TypeError):
        ops.embedding(table, idx.float())
    with pytest.raises(TypeError):
        ops.embedding(table[0], idx)
    with pytest.raises(TypeError):
        ops.embedding(table.cpu(), idx.cpu())
    with pytest.raises(IndexError):
        ops.embedding(table[:0], idx)


@pytest.mark.gpu
def test_full_size_token_and_position_lookup():
    """GPT-2's two lookups at the workload's size: 32 x 1024 tokens from [50257, 768] and 1024
    positions from [1024, 768]; every output row must be the table row it names."""
    ops = _ops()
    wte = seeded((50257, 768), seed=15, dtype=torch.bfloat16).cuda()
    wpe = seeded((1024, 768), seed=16, dtype=torch.bfloat16).cuda()
    tok = torch.randint(0, 50257, (32, 1024), device="cuda", generator=torch.Generator("cuda").manual_seed(17))
    pos = torch.arange(1024, device="cuda")
    x = ops.embedding(wte, tok)
    assert torch.equal(x, wte[tok])
    assert torch.equal(ops.embedding(wpe, pos), wpe)
    # checksum of checksums: the per-row sums of the output are the gathered per-row sums
    assert torch.equal(x.float().sum(-1), wte.float().sum(-1)[tok])


@pytest.mark.gpu
def test_graph_and_eager_surfaces_use_the_kernel():
    import torch_mojo_backend as tmb
    from torch_mojo_backend import MAPPING_TORCH_ATEN_TO_MOJO
    aten = torch.ops.aten
    assert aten.embedding in MAPPING_TORCH_ATEN_TO_MOJO

    emb = torch.nn.Embedding(100, 48).cuda().to(torch.bfloat16)
    idx = torch.randint(0, 100, (4, 7), device="cuda")
    compiled = torch.compile(emb, backend=tmb.mojo_backend, fullgraph=True)
    with torch.no_grad():
        assert torch.equal(compiled(idx), emb(idx))

    tmb.register_mojo_devices()
    w, i = emb.weight.detach().to("mojo"), idx.to("mojo")
    out = torch.nn.functional.embedding(i, w)
    assert out.device.type == "mojo" and torch.equal(out.cpu(), emb(idx).detach().cpu())
    with pytest.raises(NotImplementedError):
        torch.nn.functional.embedding(i, torch.arange(10, device="cuda").reshape(5, 2).to("mojo"))
