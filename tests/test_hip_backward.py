"""GPU parity of the backward twins (gelu, softmax / log-softmax, layer norm, linear) against the
C oracle, float64 autograd and the invariants the formulas fix."""

import numpy as np
import pytest
import torch

import oracle
from helpers import as64, seeded

pytestmark = pytest.mark.gpu

FLOATS = [torch.float32, torch.bfloat16, torch.float16]
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2, torch.float16: 3e-3}


def _ops():
    from torch_mojo_backend.eager_kernels import hip_ops
    return hip_ops


def _autograd64(fn, *inputs):
    """Gradients of sum(fn(*inputs) * g) in float64 on the CPU (inputs given in storage precision)."""
    xs = [x.double().requires_grad_(True) for x in inputs[:-1]]
    g = inputs[-1].double()
    (fn(*xs) * g).sum().backward()
    return [x.grad.numpy() for x in xs]


# ---- gelu ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("approximate", ["none", "tanh"])
@pytest.mark.parametrize("numel", [1, 7, 4096, 100003])
def test_gelu_backward(dtype, approximate, numel):
    x = seeded((numel,), seed=1, dtype=dtype) * 3
    g = seeded((numel,), seed=2, dtype=dtype)
    got = _ops().gelu_backward(g.cuda(), x.cuda(), approximate)
    assert got.dtype == dtype and got.shape == x.shape
    (want,) = _autograd64(lambda t: torch.nn.functional.gelu(t, approximate=approximate), x, g)
    scale = np.abs(as64(g)).max() + 1.0
    assert np.abs(as64(got) - want).max() <= TOL[dtype] * scale
    ref = oracle.gelu_backward(g, x, approximate)
    assert np.abs(as64(got) - as64(ref)).max() <= TOL[dtype] * scale


def test_gelu_backward_limits():
    x = torch.tensor([0.0, 30.0, -30.0, 1e4, -1e4], dtype=torch.float32)
    g = torch.full_like(x, 2.0)
    for mode in ("none", "tanh"):
        got = _ops().gelu_backward(g.cuda(), x.cuda(), mode).cpu()
        assert torch.allclose(got, torch.tensor([1.0, 2.0, 0.0, 2.0, 0.0]), atol=1e-6), (mode, got)


# ---- softmax / log-softmax ----------------------------------------------------------------------
SOFTMAX_SHAPES = [(1, 1), (3, 5), (33, 257), (64, 1024), (17, 4096), (5, 8192), (4, 50257), (2, 70000),
                  # long ragged rows: one 1024-thread workgroup per row with unaligned vectors
                  (37, 4099), (5, 16389), (6, 30001), (3, 65535), (130, 50257)]


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", SOFTMAX_SHAPES)
@pytest.mark.parametrize("log", [False, True])
def test_softmax_backward_rows(shape, dtype, log):
    x = seeded(shape, seed=3, dtype=torch.float32) * 2
    fwd = (torch.log_softmax if log else torch.softmax)(x, -1).to(dtype)
    g = seeded(shape, seed=4, dtype=dtype)
    got = _ops().softmax_backward(g.cuda(), fwd.cuda(), -1, log)
    assert got.dtype == dtype and got.shape == fwd.shape
    y64, g64 = as64(fwd), as64(g)
    if log:
        want = g64 - np.exp(y64) * g64.sum(-1, keepdims=True)
    else:
        want = y64 * (g64 - (g64 * y64).sum(-1, keepdims=True))
    # the row sum carries the fp32 error of `cols` terms of size |g| <= ~4
    bound = TOL[dtype] * (np.abs(want).max() + 1.0) + shape[1] * 2.0 ** -24 * 8.0 * (np.abs(np.exp(y64)).max() if log else 1.0)
    assert np.abs(as64(got) - want).max() <= bound
    ref = oracle.softmax_backward_rows(g, fwd, log)
    assert np.abs(as64(got) - as64(ref)).max() <= 2 * bound


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("log", [False, True])
def test_softmax_backward_long_rows_at_an_odd_address(dtype, log):
    """The saved output starts one element past a 16-byte boundary, the gradient does not: the
    long-row kernel with unaligned vector accesses."""
    rows, cols = 5, 8200
    x = seeded((rows, cols), seed=5, dtype=torch.float32) * 2
    fwd = (torch.log_softmax if log else torch.softmax)(x, -1).to(dtype)
    g = seeded((rows, cols), seed=6, dtype=dtype)
    buf = torch.zeros(rows * cols + 1, dtype=dtype, device="cuda")
    saved = buf[1:].view(rows, cols)
    saved.copy_(fwd)
    assert saved.data_ptr() % 16 != 0
    got = _ops().softmax_backward(g.cuda(), saved, -1, log)
    ref = oracle.softmax_backward_rows(g, fwd, log)
    bound = TOL[dtype] * (np.abs(as64(ref)).max() + 1.0) + cols * 2.0 ** -24 * 16.0
    assert np.abs(as64(got) - as64(ref)).max() <= bound


def test_softmax_backward_invariants_and_dims():
    # a constant upstream gradient cancels (softmax) / the row of gradients sums to zero (log)
    x = seeded((6, 300), seed=5)
    y = torch.softmax(x, -1)
    got = _ops().softmax_backward(torch.full_like(y, 3.0).cuda(), y.cuda(), -1, False).cpu()
    assert got.abs().max().item() <= 1e-6
    ly = torch.log_softmax(x, -1)
    g = seeded((6, 300), seed=6)
    got = _ops().softmax_backward(g.cuda(), ly.cuda(), -1, True).cpu()
    assert got.sum(-1).abs().max().item() <= 1e-4
    # other dims go through a transposed copy
    x3 = seeded((4, 9, 11), seed=7)
    g3 = seeded((4, 9, 11), seed=8)
    for dim in (0, 1, -1):
        xr = x3.clone().requires_grad_(True)
        out = torch.softmax(xr, dim)
        out.backward(g3)
        got = _ops().softmax_backward(g3.cuda(), out.detach().cuda(), dim, False).cpu()
        torch.testing.assert_close(got, xr.grad, rtol=1e-5, atol=1e-6)


# ---- cross-entropy: NLL backward + log-softmax backward in one pass ------------------------------
LOSS_SHAPES = [(1, 5), (7, 64), (33, 1000), (64, 4104), (19, 50257), (300, 257), (5, 8200)]


def _loss_case(shape, dtype, seed):
    rows, cols = shape
    x = seeded(shape, seed=seed, dtype=torch.float32) * 3
    logp = torch.log_softmax(x, -1).to(dtype)
    g = torch.Generator().manual_seed(seed + 1)
    target = torch.randint(0, cols, (rows,), generator=g)
    target[::5] = -100                       # ignored rows
    if rows > 2:
        target[1], target[2] = 0, cols - 1   # first and last class
    return logp, target


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", LOSS_SHAPES)
@pytest.mark.parametrize("reduction", [0, 1, 2])
def test_nll_log_softmax_backward(shape, dtype, reduction):
    rows, cols = shape
    logp, target = _loss_case(shape, dtype, seed=13)
    valid = int((target != -100).sum())
    total_weight = torch.tensor(float(max(valid, 1)), dtype=dtype)
    grad_out = (seeded((rows,), seed=15).abs() + 0.5).to(dtype) if reduction == 0 \
        else torch.tensor(0.75, dtype=dtype)
    got = _ops().nll_log_softmax_backward(grad_out.cuda(), logp.cuda(), target.cuda(),
                                          total_weight.cuda(), reduction, -100)
    assert got.dtype == dtype and tuple(got.shape) == shape
    # float64 closed form: w * (softmax - onehot), zero rows where the target is ignored
    p = np.exp(as64(logp))
    w = as64(grad_out) if reduction == 0 else np.full(rows, float(grad_out))
    if reduction == 1:
        w = w / float(total_weight)
    onehot = np.zeros(shape)
    keep = (target != -100).numpy()
    onehot[np.arange(rows)[keep], target.numpy()[keep]] = 1.0
    want = (w * keep)[:, None] * (p - onehot)
    bound = 2 * TOL[dtype] * (np.abs(want).max() + np.abs(w).max())
    assert np.abs(as64(got) - want).max() <= bound
    # the C restatement of the reference's two kernels
    ref = oracle.nll_log_softmax_backward(grad_out, logp, target, total_weight, reduction, -100)
    assert np.abs(as64(got) - as64(ref)).max() <= bound
    # and, bit for bit, the two kernels this pass stands for
    dense = torch.ops.aten.nll_loss_backward(grad_out.cuda(), logp.cuda(), target.cuda(), None, reduction,
                                             -100, total_weight.cuda())
    two = _ops().softmax_backward(dense, logp.cuda(), -1, True)
    if dtype == torch.float16:
        # (fp16 only: the compiler may fold the last multiply-add into the conversion, one rounding
        # instead of two, in one kernel and not in the other: a unit in the last place, rarely)
        differ = got != two
        assert int(differ.sum()) <= max(1, got.numel() // 1000)
        assert ((got.double() - two.double()).abs() <= 2.0 ** -10 * two.double().abs() + 1e-12).all()
    else:
        assert torch.equal(got, two)
    # rows of whole 16-byte vectors with zeros behind the last class
    unit = 16 // logp.element_size()
    if cols % unit:
        assert got.stride(0) == (cols + 63) // 64 * 64 and got.stride(0) % unit == 0
        whole = got.as_strided((rows, got.stride(0)), (got.stride(0), 1), got.storage_offset())
        assert float(whole[:, cols:].abs().max()) == 0.0
    else:
        assert got.is_contiguous()


def test_nll_log_softmax_backward_reads_strided_rows_and_feeds_the_products():
    """Log-probabilities that are a column slice of something wider (pitch > classes), and the
    products that take the result as an operand: the padded buffer is found instead of copied."""
    rows, cols, hidden = 2048, 50257, 64
    wide = torch.log_softmax(seeded((rows, cols + 3), seed=21) * 2, -1).bfloat16().cuda()
    logp = wide[:, 1:cols + 1]
    target = torch.randint(0, cols, (rows,), generator=torch.Generator().manual_seed(3)).cuda()
    one, tw = torch.tensor(1.0).bfloat16().cuda(), torch.tensor(float(rows)).bfloat16().cuda()
    ops = _ops()
    copies = []
    plain_copy = ops._pad_last_copy

    def counting(t, size):
        copies.append((tuple(t.shape), size))
        return plain_copy(t, size)

    w = (seeded((cols, hidden), seed=22) * 0.05).bfloat16().cuda()
    x = seeded((rows, hidden), seed=23).bfloat16().cuda()
    before = ops.pad_reuse_begin()
    ops._pad_last_copy = counting
    try:
        dl = ops.nll_log_softmax_backward(one, logp, target, tw, 1, -100)
        dx = ops.gemm(dl, w)            # contracts over the classes
        dw = ops.gemm(dl.t(), x)        # has them as its transposed dimension
        torch.cuda.synchronize()
    finally:
        ops._pad_last_copy = plain_copy
        ops.pad_reuse_end(before)
    assert not [c for c in copies if c[0] == (rows, cols)], copies
    ref = oracle.nll_log_softmax_backward(one.cpu(), logp.cpu().contiguous(), target.cpu(), tw.cpu(), 1, -100)
    assert torch.equal(dl.cpu(), ref) or (dl.cpu().double() - ref.double()).abs().max() <= 2.0 ** -8 / rows
    for got, want in ((dx, ref.double() @ w.cpu().double()), (dw, ref.double().t() @ x.cpu().double())):
        err = (got.cpu().double() - want).norm() / want.norm()
        assert err < 4e-3, err


# ---- layer norm ---------------------------------------------------------------------------------
LN_SHAPES = [(1, 8), (5, 65), (33, 768), (64, 1000), (9, 4096), (300, 768), (7, 12288), (3, 50257)]


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", LN_SHAPES)
@pytest.mark.parametrize("affine", [True, False])
def test_layer_norm_backward(shape, dtype, affine):
    rows, cols = shape
    x = seeded(shape, seed=9, dtype=dtype)
    g = seeded(shape, seed=10, dtype=dtype)
    w = (1 + 0.1 * seeded((cols,), seed=11)).to(dtype) if affine else None
    out, mean, rstd = _ops().layer_norm(x.cuda(), [cols], None if w is None else w.cuda(), None, 1e-5)
    dx, dw, db = _ops().layer_norm_backward(g.cuda(), x.cuda(), [cols], mean, rstd,
                                            None if w is None else w.cuda(), [True, affine, True])
    assert dx.dtype == dtype and dx.shape == x.shape and db.shape == (cols,)
    x64 = x.double().requires_grad_(True)
    w64 = None if w is None else w.double().requires_grad_(True)
    b64 = torch.zeros(cols, dtype=torch.float64, requires_grad=True)
    (torch.nn.functional.layer_norm(x64, [cols], w64, b64, 1e-5) * g.double()).sum().backward()
    scale = np.abs(x64.grad.numpy()).max() + 1.0
    assert np.abs(as64(dx) - x64.grad.numpy()).max() <= TOL[dtype] * scale * 4
    col_tol = TOL[dtype] * (np.abs(b64.grad.numpy()).max() + 1.0) + rows * 2.0 ** -22
    assert np.abs(as64(db) - b64.grad.numpy()).max() <= col_tol * 4
    if affine:
        assert np.abs(as64(dw) - w64.grad.numpy()).max() <= \
            (TOL[dtype] * (np.abs(w64.grad.numpy()).max() + 1.0) + rows * 2.0 ** -22) * 4
    rdx, rdw, rdb = oracle.layer_norm_backward_rows(g, x, mean.cpu(), rstd.cpu(), w)
    assert np.abs(as64(dx) - as64(rdx)).max() <= TOL[dtype] * scale * 4
    assert np.abs(as64(db) - as64(rdb)).max() <= col_tol * 4


def test_layer_norm_backward_invariants_and_masks():
    x = seeded((40, 512), seed=12)
    g = seeded((40, 512), seed=13)
    w = 1 + 0.1 * seeded((512,), seed=14)
    _, mean, rstd = _ops().layer_norm(x.cuda(), [512], w.cuda(), None, 1e-5)
    dx, dw, db = _ops().layer_norm_backward(g.cuda(), x.cuda(), [512], mean, rstd, w.cuda(),
                                            [True, False, False])
    assert dw is None and db is None
    dx = dx.cpu()
    xhat = (x - x.mean(-1, keepdim=True)) * rstd.cpu().view(-1, 1)
    # grad_input is orthogonal to the constant vector and to xhat
    assert dx.sum(-1).abs().max().item() <= 2e-4
    assert (dx * xhat).sum(-1).abs().max().item() <= 2e-3
    only_params = _ops().layer_norm_backward(g.cuda(), x.cuda(), [512], mean, rstd, w.cuda(),
                                             [False, True, True])
    assert only_params[0] is None
    torch.testing.assert_close(only_params[2].cpu(), g.sum(0), rtol=1e-5, atol=1e-4)
    # same call twice: bit-identical parameter gradients (fixed summation order)
    again = _ops().layer_norm_backward(g.cuda(), x.cuda(), [512], mean, rstd, w.cuda(),
                                       [False, True, True])
    assert torch.equal(only_params[1], again[1]) and torch.equal(only_params[2], again[2])


LN_ADD_SHAPES = [(5, 64), (33, 768), (300, 768), (1030, 1024), (64, 1000), (9, 4096), (70, 2048),
                 (40, 8192), (7, 12288)]


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("shape", LN_ADD_SHAPES)
@pytest.mark.parametrize("form", ["add+sum", "add", "sum"])
def test_layer_norm_backward_add(shape, dtype, form):
    """grad_input + addend and its column sums in the layer-norm backward's own pass: the same
    values as the three separate steps (bit for bit in bfloat16 and float32; float16 may round an
    element the other way where the compiler folds the conversion into the multiply)."""
    rows, cols = shape
    ops = _ops()
    x = seeded(shape, seed=31, dtype=dtype).cuda()
    g = seeded(shape, seed=32, dtype=dtype).cuda()
    a = seeded(shape, seed=33, dtype=dtype).cuda() if "add" in form else None
    w = (1 + 0.1 * seeded((cols,), seed=34)).to(dtype).cuda()
    _, mean, rstd = ops.layer_norm(x, [cols], w, None, 1e-5)
    got = ops.layer_norm_backward_add(g, x, [cols], mean, rstd, w, a, "sum" in form)
    epv = 16 // x.element_size()
    covered = cols % epv == 0 and cols // epv <= (2048 if dtype == torch.float32 else 1024)
    if not covered:
        assert got is None
        return
    dx, dw, db, ds = got
    rdx, rdw, rdb = ops.layer_norm_backward(g, x, [cols], mean, rstd, w, [True, True, True])
    want = rdx if a is None else rdx + a
    if dtype == torch.float16:
        off = (dx != want)
        assert off.float().mean().item() <= 1e-3
        assert (dx.double() - want.double()).abs().max().item() <= \
            2.0 ** -10 * (want.double().abs().max().item() + 1.0)
    else:
        assert torch.equal(dx, want)
    for mine, theirs in ((dw, rdw), (db, rdb)):
        scale = theirs.double().abs().max().item() + 1.0
        assert (mine.double() - theirs.double()).abs().max().item() <= TOL[dtype] * scale
    if "sum" in form:
        ref = dx.double().sum(0)
        bound = TOL[dtype] * (ref.abs().max().item() + 1.0) + rows * 2.0 ** -22 * dx.double().abs().max().item()
        assert ds.shape == (cols,) and ds.dtype == dtype
        assert (ds.double() - ref).abs().max().item() <= 4 * bound
    else:
        assert ds is None
    # against the CPU restatement of the layer-norm backward, with the add and its two roundings
    odx, _, _ = oracle.layer_norm_backward_rows(g.cpu(), x.cpu(), mean.cpu(), rstd.cpu(), w.cpu())
    owant = odx if a is None else (odx + a.cpu())
    scale = owant.double().abs().max().item() + 1.0
    assert (dx.cpu().double() - owant.double()).abs().max().item() <= TOL[dtype] * scale * 4


def test_layer_norm_backward_add_rejects_what_it_cannot_mean():
    ops = _ops()
    x = seeded((8, 64), seed=35).cuda()
    _, mean, rstd = ops.layer_norm(x, [64], None, None, 1e-5)
    with pytest.raises(ValueError):
        ops.layer_norm_backward_add(x, x, [64], mean, rstd, None, None, False)
    with pytest.raises(ValueError):
        ops.layer_norm_backward_add(x, x, [64], mean, rstd, None, x[:4], True)
    from torch_mojo_backend import eager_kernels
    lib = eager_kernels.lib()
    assert lib.tmb_layer_norm_backward_add_workspace_bytes(8, 63, 0) == 0
    rc = lib.tmb_layer_norm_backward_add_rows(x.data_ptr(), x.data_ptr(), x.data_ptr(), None, x.data_ptr(),
                                              x.data_ptr(), mean.data_ptr(), rstd.data_ptr(), None, None,
                                              8, 64, 0, None, 0, None)
    assert rc == -1  # neither an addend nor the column sums


# ---- linear -------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [((4, 33, 64), 48), ((512, 768), 2304), ((8, 128, 768), 768)])
def test_linear_backward(shape, dtype):
    xshape, out_f = shape
    in_f = xshape[-1]
    x = seeded(xshape, seed=15, dtype=dtype)
    w = (seeded((out_f, in_f), seed=16) * 0.05).to(dtype)
    g = seeded(xshape[:-1] + (out_f,), seed=17, dtype=dtype)
    dx, dw, db = _ops().linear_backward(x.cuda(), g.cuda(), w.cuda(), [True, True, True])
    x64, w64 = x.double().requires_grad_(True), w.double().requires_grad_(True)
    b64 = torch.zeros(out_f, dtype=torch.float64, requires_grad=True)
    (torch.nn.functional.linear(x64, w64, b64) * g.double()).sum().backward()
    rel = 1e-5 if dtype == torch.float32 else 1e-2
    for got, want in ((dx, x64.grad), (dw, w64.grad), (db, b64.grad)):
        want = want.numpy()
        assert np.linalg.norm(as64(got) - want) <= rel * np.linalg.norm(want) + 1e-6
    none_x = _ops().linear_backward(x.cuda(), g.cuda(), w.cuda(), [False, True, False])
    assert none_x[0] is None and none_x[1] is not None and none_x[2].abs().sum().item() == 0
