"""GPU parity of sum / mean / amax / argmax against the CPU oracle and float64 closed forms."""

import numpy as np
import pytest
import torch

import oracle
from oracle import closed_form as cf
from helpers import as64, assert_close64, seeded

pytestmark = pytest.mark.gpu

FLOATS = [torch.float32, torch.bfloat16, torch.float16]


def _ops():
    from torch_mojo_backend.eager_kernels import hip_ops
    return hip_ops


def _ek():
    from torch_mojo_backend import eager_kernels
    return eager_kernels


def _dev(t):
    return t.to("cuda")


# (rows, cols): wave-per-row, block-per-row, split rows, unaligned widths, a single long row.
REDUCE_SHAPES = [(1, 1), (5, 3), (64, 64), (33, 257), (1000, 768), (2048, 4096), (300, 4097),
                 (7, 50257), (3, 100003), (1, 1 << 20), (1, (1 << 22) + 5), (2, 300000)]


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", REDUCE_SHAPES)
def test_sum_mean_amax_rows(shape, dtype):
    x = seeded(shape, seed=shape[1] % 997, dtype=dtype)
    xd = _dev(x)
    x64 = as64(x)
    bound = cf.sum_error_bound(x64, axis=-1)
    n = shape[1]
    s = _ops().reduce(xd, [1], False, _ek().SUM)
    assert s.dtype == dtype and tuple(s.shape) == (shape[0],)
    assert_close64(s, x64.sum(-1), extra_abs=bound, what=f"sum {shape}")
    m = _ops().reduce(xd, [1], False, _ek().MEAN)
    assert_close64(m, x64.mean(-1), extra_abs=bound / n, what=f"mean {shape}")
    a = _ops().reduce(xd, [1], False, _ek().AMAX)
    assert np.array_equal(as64(a), x64.max(-1)), "amax must be exact"
    # C restatement of the reference kernel (sequential fp32): same bound applies to it
    ref = oracle.reduce_rows(x, oracle.SUM)
    assert_close64(s, as64(ref), extra_abs=2 * bound, rounded_want=True, what="sum vs C oracle")


@pytest.mark.parametrize("dims,keepdim", [([0], False), ([1], True), ([0, 2], False), ([2], True),
                                          ([0, 1, 2], False), ([0, 1, 2], True), ([1, 2], False)])
def test_reduce_dims_and_keepdim(dims, keepdim):
    x = seeded((6, 10, 12), seed=4)
    for op, ref in ((_ek().SUM, torch.sum), (_ek().MEAN, torch.mean), (_ek().AMAX, torch.amax)):
        got = _ops().reduce(_dev(x), dims, keepdim, op)
        want = ref(x, dim=dims, keepdim=keepdim)
        assert got.shape == want.shape
        torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-5)


def test_full_reduction_benchmark_size_properties():
    """[65536, 4096] fp32 (the benchmark tensor): linearity and a sum of row sums."""
    g = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(65536, 4096, generator=g, device="cuda")
    ops, ek = _ops(), _ek()
    total = ops.reduce(x, [0, 1], False, ek.SUM)
    rows = ops.reduce(x, [1], False, ek.SUM)
    total_of_rows = ops.reduce(rows, [0], False, ek.SUM)
    exact = x.double().sum().item()
    l1 = x.double().abs().sum().item()
    assert abs(total.item() - exact) <= 1e-6 * l1 * 1e-1 + 1e-5 * abs(exact)
    assert abs(total_of_rows.item() - exact) <= 1e-6 * l1 * 1e-1 + 1e-5 * abs(exact)
    # bit-reproducible: same launch twice, identical bits
    again = ops.reduce(x, [0, 1], False, ek.SUM)
    assert total.view(torch.int32).item() == again.view(torch.int32).item()
    # mean = sum / numel, amax exact
    mean = ops.reduce(x, [0, 1], False, ek.MEAN)
    assert abs(mean.item() - exact / x.numel()) <= 1e-6
    assert ops.reduce(x, [0, 1], False, ek.AMAX).item() == x.max().item()
    # linearity: sum(2x) == 2 sum(x) exactly (scaling by 2 is exact in fp32)
    assert ops.reduce(x * 2, [0, 1], False, ek.SUM).item() == 2 * total.item()


def test_amax_propagates_nan_and_handles_inf():
    x = seeded((4, 5000), seed=3)
    x[1, 4321] = float("nan")
    x[2, 17] = float("inf")
    x[3, :] = float("-inf")
    got = _ops().reduce(_dev(x), [1], False, _ek().AMAX).cpu()
    want = torch.amax(x, dim=1)
    assert torch.isnan(got[1]) and got[2] == float("inf") and got[3] == float("-inf")
    assert got[0] == want[0]


def test_integer_reductions_are_exact():
    g = torch.Generator().manual_seed(7)
    x = torch.randint(-2 ** 40, 2 ** 40, (37, 5001), generator=g, dtype=torch.int64)
    assert torch.equal(_ops().reduce(_dev(x), [1], False, _ek().SUM).cpu(), x.sum(1))
    assert torch.equal(_ops().reduce(_dev(x), [1], False, _ek().AMAX).cpu(), x.amax(1))
    assert torch.equal(_ops().reduce(_dev(x), [0, 1], False, _ek().SUM).cpu(), x.sum())
    xi = torch.randint(-2 ** 31, 2 ** 31 - 1, (3, 70001), generator=g, dtype=torch.int32)
    assert torch.equal(_ops().reduce(_dev(xi), [1], False, _ek().AMAX).cpu(), xi.amax(1))
    assert torch.equal(_ops().argmax(_dev(xi), 1, False).cpu(), xi.argmax(1))
    assert torch.equal(_ops().argmax(_dev(x), 1, False).cpu(), x.argmax(1))


def _logits_with_ties(rows=512, cols=50257, seed=0):
    """Benchmark logits: 1% of rows carry an injected tie above the row maximum."""
    x = seeded((rows, cols), seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    n_tied = max(1, -(-rows // 100))
    tied_rows = torch.randperm(rows, generator=g)[: n_tied + 2].tolist()
    expected = {}
    for r in tied_rows[:n_tied]:
        j = sorted(torch.randint(0, cols, (2,), generator=g).tolist())
        if j[0] == j[1]:
            j[1] = (j[0] + 1) % cols
            j.sort()
        x[r, j[0]] = x[r, j[1]] = x[r].max() + 1
        expected[r] = j[0]
    r3, rl = tied_rows[n_tied], tied_rows[n_tied + 1]
    top = x[r3].max() + 1
    x[r3, 0] = x[r3, cols // 2] = x[r3, cols - 1] = top   # three-way tie including column 0
    expected[r3] = 0
    top = x[rl].max() + 1
    x[rl, cols - 2] = x[rl, cols - 1] = top               # tie at the very end of the row
    expected[rl] = cols - 2
    return x, expected


@pytest.mark.parametrize("dtype", FLOATS)
def test_argmax_vocab_with_ties_is_bit_exact(dtype):
    x, expected = _logits_with_ties()
    x = x.to(dtype)
    got = _ops().argmax(_dev(x), -1, False)
    assert got.dtype == torch.int64
    got = got.cpu()
    assert torch.equal(got, oracle.argmax_rows(x))
    assert torch.equal(got, torch.argmax(x, dim=-1))
    if dtype == torch.float32:
        for r, j in expected.items():
            assert got[r].item() == j


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (64, 64), (257, 1000), (5, 65537), (2, 1 << 21),
                                   (256, 40001), (300, 70003),  # one wide workgroup per row
                                   (1, (1 << 23) + 3)])
def test_argmax_shapes(shape):
    x = seeded(shape, seed=shape[1] % 991)
    x[:, shape[1] // 2] = x.max() + 1  # a planted maximum, as the reference's vocab test does
    if shape[1] > 2:
        x[0, shape[1] - 1] = x.max()   # and a tie with a later column in row 0
    got = _ops().argmax(_dev(x), 1, False).cpu()
    assert torch.equal(got, torch.argmax(x, dim=1))
    assert torch.equal(got, oracle.argmax_rows(x))


# Rows of at least 2048 floating-point columns are cut into work units of 256 lanes, one 16-byte
# vector at a time per lane; the cases below sit on every seam of that scheme: unit boundaries,
# elements in front of / behind the whole vectors of a unit (odd pitches), units with a single
# vector per lane and with seven, rows of exactly one unit, storage offsets.
VEC_SHAPES = [(3, 2048), (5, 2049), (7, 4099), (2, 7168), (2, 7169), (4, 7233), (33, 14336), (9, 14337),
              (512, 50257), (300, 57344), (257, 57347), (256, 2048), (260, 28673), (32, 50257), (1, 50257), (2048, 6151), (1, 1 << 20), (3, (1 << 21) + 5)]


def _argmax_adversarial(shape, dtype, seed):
    rows, cols = shape
    x = seeded(shape, seed=seed).to(dtype)
    g = torch.Generator().manual_seed(seed + 7)
    pick = lambda n: torch.randint(0, cols, (n,), generator=g).tolist()   # noqa: E731
    top = float(x.float().max()) + 1
    for r in range(rows):
        kind = r % 16
        if kind == 0:      # tie between two random columns
            a = pick(2)
            x[r, a] = top
        elif kind == 1:    # maximum in the first / last column
            x[r, 0] = top
        elif kind == 2:
            x[r, cols - 1] = top
        elif kind == 3:    # two NaN: the first wins, whatever else the row holds
            a = pick(2)
            x[r, a] = float("nan")
            x[r, pick(1)] = float("inf")
        elif kind == 4:    # the whole row equal
            x[r] = 0.75
        elif kind == 5:    # all -inf
            x[r] = float("-inf")
        elif kind == 6:    # -inf everywhere but one finite value
            x[r] = float("-inf")
            x[r, pick(1)] = -3.0
        elif kind == 7:    # +inf twice, and a -inf (the sum check fires without any NaN)
            a = pick(3)
            x[r, a[:2]] = float("inf")
            x[r, a[2]] = float("-inf")
        elif kind == 8:    # zeros of both signs tie
            x[r] = -0.0
            x[r, pick(1)] = 0.0
        elif kind == 9:    # NaN in the last column only
            x[r, cols - 1] = float("nan")
        elif kind == 10:   # a tie that straddles a unit boundary (units are multiples of 64 wide)
            j = min(cols - 1, (cols // 2) // 64 * 64)
            x[r, max(j - 1, 0)] = top
            x[r, j] = top
        elif kind == 11:   # negative NaN (sign bit set), as 0/0 produces on the host
            x[r, pick(1)] = -float("nan")
    return x


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", VEC_SHAPES)
def test_argmax_vector_units_are_bit_exact(shape, dtype):
    x = _argmax_adversarial(shape, dtype, seed=shape[1] % 977)
    want = torch.argmax(x, dim=1)
    got = _ops().argmax(_dev(x), 1, False).cpu()
    bad = (got != want).nonzero().flatten().tolist()
    assert not bad, f"{shape} {dtype}: rows {bad[:8]} got {got[bad[:8]].tolist()} want {want[bad[:8]].tolist()}"
    if shape[0] * shape[1] <= 1 << 22:
        assert torch.equal(got, oracle.argmax_rows(x))


@pytest.mark.parametrize("dtype", FLOATS)
def test_argmax_rows_that_start_anywhere(dtype):
    """A view whose rows start 1 .. 9 elements into 16-byte vectors (storage offset, odd pitch)."""
    base = seeded((6, 9001), seed=5).to(dtype)
    for offset in (1, 2, 3, 5, 9):
        flat = torch.zeros(6 * 9001 + offset, dtype=dtype)
        flat[offset:] = base.reshape(-1)
        dev = _dev(flat)[offset:].view(6, 9001)
        assert dev.data_ptr() % 16 != 0 or offset * base.element_size() % 16 == 0
        assert torch.equal(_ops().argmax(dev, 1, False).cpu(), torch.argmax(base, dim=1))


def test_argmax_workspace_is_what_the_entry_point_asks_for():
    ek = _ek()
    L = ek.lib()
    stream = torch.cuda.current_stream().cuda_stream
    # at least a row per CU of fp32 rows that a workgroup holds: whole rows, one launch, no workspace
    assert L.tmb_argmax_workspace_bytes(512, 50257, ek.F32) == 0
    x = _dev(seeded((512, 50257), seed=1))
    out = torch.empty(512, dtype=torch.int64, device=x.device)
    assert L.tmb_argmax_rows(out.data_ptr(), x.data_ptr(), 512, 50257, ek.F32, None, 0, stream) == 0
    assert torch.equal(out.cpu(), torch.argmax(x.cpu(), dim=1))
    # fewer rows: units of a row and a combining launch, 16 bytes per unit
    need = L.tmb_argmax_workspace_bytes(128, 50257, ek.F32)
    assert need > 0 and need % (128 * 16) == 0
    assert L.tmb_argmax_workspace_bytes(512, 50257, ek.I64) == L.tmb_reduce_workspace_bytes(512, 50257, ek.I64)
    assert L.tmb_argmax_workspace_bytes(4096, 4096, ek.F32) == 0        # one unit per row
    assert L.tmb_argmax_workspace_bytes(0, 4096, ek.F32) == 0
    small = torch.empty(need - 16, dtype=torch.uint8, device=x.device)
    assert L.tmb_argmax_rows(out.data_ptr(), x.data_ptr(), 128, 50257, ek.F32, small.data_ptr(),
                             need - 16, stream) == ek.ERR_WORKSPACE
    assert L.tmb_argmax_rows(out.data_ptr(), x.data_ptr(), 128, 50257, ek.F32, None, 0, stream) == ek.ERR_WORKSPACE
    full = torch.empty(need, dtype=torch.uint8, device=x.device)
    assert L.tmb_argmax_rows(out.data_ptr(), x.data_ptr(), 128, 50257, ek.F32, full.data_ptr(), need, stream) == 0
    assert torch.equal(out[:128].cpu(), torch.argmax(x[:128].cpu(), dim=1))


def test_argmax_dim_none_keepdim_and_nan():
    x = seeded((7, 9, 11), seed=8)
    ops = _ops()
    assert torch.equal(ops.argmax(_dev(x), None, False).cpu(), torch.argmax(x))
    assert ops.argmax(_dev(x), None, True).shape == (1, 1, 1)
    for d in (0, 1, 2, -1):
        for keep in (False, True):
            assert torch.equal(ops.argmax(_dev(x), d, keep).cpu(), torch.argmax(x, dim=d, keepdim=keep))
    x[2, 3, 5] = float("nan")
    x[2, 3, 7] = float("nan")
    assert torch.equal(ops.argmax(_dev(x), 2, False).cpu(), torch.argmax(x, dim=2))
    all_equal = torch.zeros(3, 70000)
    assert torch.equal(ops.argmax(_dev(all_equal), 1, False).cpu(), torch.zeros(3, dtype=torch.int64))


# ---- reductions over the leading dimension (bias gradients, sum(x, dim=0)) ---------------------
# (rows, cols): one slab and many, whole vectors and ragged widths, the bias-gradient shapes of
# GPT-2 (tokens x 768 / 2304 / 3072), a width of one, more columns than rows
COLS_SHAPES = [(16, 1024), (17, 1031), (4096, 768), (16384, 2304), (2048, 3072), (100000, 8),
               (50000, 1), (33, 50257), (30000, 5)]


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", COLS_SHAPES)
def test_sum_mean_amax_over_the_leading_dimension(shape, dtype):
    x = seeded(shape, seed=shape[0] % 991, dtype=dtype)
    assert x.numel() >= _ops()._COLS_KERNEL_MIN_ELEMENTS
    xd, x64 = _dev(x), as64(x)
    bound = cf.sum_error_bound(x64.T, axis=-1)
    s = _ops().reduce(xd, [0], False, _ek().SUM)
    assert s.dtype == dtype and tuple(s.shape) == (shape[1],)
    assert_close64(s, x64.sum(0), extra_abs=bound, what=f"sum {shape}")
    m = _ops().reduce(xd, [0], True, _ek().MEAN)
    assert tuple(m.shape) == (1, shape[1])
    assert_close64(m[0], x64.mean(0), extra_abs=bound / shape[0], what=f"mean {shape}")
    a = _ops().reduce(xd, [0], False, _ek().AMAX)
    assert np.array_equal(as64(a), x64.max(0)), "amax must be exact"
    # the C restatement works on rows: hand it the transposed matrix
    ref = oracle.reduce_rows(x.t().contiguous(), oracle.SUM)
    assert_close64(s, as64(ref), extra_abs=2 * bound, rounded_want=True, what="sum vs C oracle")
    # same call, same bits (fixed order of additions)
    assert torch.equal(s, _ops().reduce(xd, [0], False, _ek().SUM))


def test_leading_dimension_reductions_of_higher_rank_nan_and_views():
    x = seeded((12, 50, 40, 16), seed=7)
    for dims in ([0], [0, 1], [0, 1, 2]):
        got = _ops().reduce(_dev(x), dims, False, _ek().SUM)
        assert_close64(got, as64(x).sum(tuple(dims)), extra_abs=cf.sum_error_bound(
            np.moveaxis(as64(x), dims, [-1 - i for i in range(len(dims))]).reshape(*x.shape[len(dims):], -1), axis=-1))
        assert tuple(_ops().reduce(_dev(x), dims, True, _ek().AMAX).shape) == tuple(
            1 if d in dims else x.shape[d] for d in range(4))
    y = seeded((5000, 24), seed=8)
    y[1234, 7] = float("nan")
    y[4000, 3] = float("inf")
    a = _ops().reduce(_dev(y), [0], False, _ek().AMAX).cpu()
    assert torch.isnan(a[7]) and a[3] == float("inf") and not torch.isnan(a[[0, 1, 2]]).any()
    # a view that is not contiguous, and an integer tensor, keep the transposing route
    z = _dev(seeded((300, 128), seed=9))
    assert_close64(_ops().reduce(z[:, ::2], [0], False, _ek().SUM), as64(z.cpu())[:, ::2].sum(0), atol=1e-3)
    i = torch.arange(40000, dtype=torch.int64).reshape(2000, 20)
    assert torch.equal(_ops().reduce(_dev(i), [0], False, _ek().SUM).cpu(), i.sum(0))


def test_reduce_cols_entry_point_checks_its_workspace():
    ek = _ek()
    L = ek.lib()
    x = _dev(seeded((4096, 768), seed=1))
    out = torch.empty(768, device="cuda")
    need = L.tmb_reduce_cols_workspace_bytes(4096, 768, ek.F32)
    assert need >= 768 * 4
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    assert L.tmb_reduce_cols(out.data_ptr(), x.data_ptr(), 4096, 768, ek.SUM, ek.F32, ws.data_ptr(), need - 1, st) == -3
    assert L.tmb_reduce_cols(out.data_ptr(), x.data_ptr(), 4096, 768, ek.SUM, ek.F32, None, 0, st) == -3
    assert L.tmb_reduce_cols(out.data_ptr(), x.data_ptr(), 0, 768, ek.SUM, ek.F32, None, 0, st) == -2
    assert L.tmb_reduce_cols(out.data_ptr(), x.data_ptr(), 4096, 768, 7, ek.F32, ws.data_ptr(), need, st) == -1
    assert L.tmb_reduce_cols(out.data_ptr(), x.data_ptr(), 4096, 768, ek.SUM, ek.I64, ws.data_ptr(), need, st) == -2
    assert L.tmb_reduce_cols(out.data_ptr(), x.data_ptr(), 4096, 768, ek.SUM, ek.F32, ws.data_ptr(), need, st) == 0
    assert_close64(out, as64(x.cpu()).sum(0), atol=2e-3)


def test_read_only_yardstick_reads_and_writes_nothing():
    """tmb_read_bytes: the bandwidth yardstick beside the reductions. It must leave its sink
    alone on ordinary data and refuse what it cannot read as 16-byte vectors."""
    ek = _ek()
    L = ek.lib()
    x = _dev(seeded((1024, 1031), seed=3))
    sink = torch.full((4,), 12345, dtype=torch.int32, device=x.device)
    stream = torch.cuda.current_stream().cuda_stream
    assert L.tmb_read_bytes(x.data_ptr(), x.numel() * 4, sink.data_ptr(), stream) == 0
    assert L.tmb_read_bytes(x.data_ptr(), 8, sink.data_ptr(), stream) == 0          # less than a vector
    torch.cuda.synchronize()
    assert sink.cpu().tolist() == [12345] * 4
    assert L.tmb_read_bytes(None, 1024, sink.data_ptr(), stream) == ek.ERR_INVALID_ARGUMENT
    assert L.tmb_read_bytes(x.data_ptr(), 1024, None, stream) == ek.ERR_INVALID_ARGUMENT
    assert L.tmb_read_bytes(x.data_ptr() + 4, 1024, sink.data_ptr(), stream) == ek.ERR_UNSUPPORTED
