"""tmb_reduce_rows_static — the entry point that allocates nothing — through the C ABI, against
tmb_reduce_rows with a caller-provided workspace. Both run the same kernels with the same
partition, so every result must be bit-identical; two calls in a row share the library's static
scratch array, the second with a smaller input."""

import ctypes

import pytest
import torch

STATIC_SCRATCH_BYTES = 256 * 1024


def _both(x2d, op, ek):
    L = ek.lib()
    rows, cols = x2d.shape
    code = {torch.float32: ek.F32, torch.bfloat16: ek.BF16, torch.float16: ek.F16,
            torch.int64: ek.I64}[x2d.dtype]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    need = L.tmb_reduce_workspace_bytes(rows, cols, code)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=x2d.device)
    want = torch.full((rows,), 7, dtype=x2d.dtype, device=x2d.device)
    got = torch.full((rows,), 9, dtype=x2d.dtype, device=x2d.device)
    rc = L.tmb_reduce_rows(want.data_ptr(), x2d.data_ptr(), rows, cols, op, code, ws.data_ptr(),
                           need, stream)
    assert rc == 0, ek.status_string(rc)
    rc = L.tmb_reduce_rows_static(got.data_ptr(), x2d.data_ptr(), rows, cols, op, code, stream)
    assert rc == 0, ek.status_string(rc)
    torch.cuda.synchronize()
    return got, want, need


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_calls_in_a_row_share_the_static_scratch(dtype):
    from torch_mojo_backend import eager_kernels as ek

    g = torch.Generator().manual_seed(0)
    big = torch.randn(3, 1_500_000, generator=g).to(dtype).cuda()      # split: partials in scratch
    small = torch.randn(2, 70_001, generator=g).to(dtype).cuda()       # fewer, shorter partials
    for op in (ek.SUM, ek.MEAN, ek.AMAX):
        got, want, need = _both(big, op, ek)
        assert need > 0
        assert torch.equal(got.view(torch.int32 if dtype == torch.float32 else torch.int16),
                           want.view(torch.int32 if dtype == torch.float32 else torch.int16))
        got2, want2, need2 = _both(small, op, ek)
        assert 0 < need2 < need
        assert torch.equal(got2.view(torch.int32 if dtype == torch.float32 else torch.int16),
                           want2.view(torch.int32 if dtype == torch.float32 else torch.int16))
    # against the mathematics as well: a float64 sum of the same values
    got, _, _ = _both(big, ek.SUM, ek)
    ref = big.double().sum(dim=1)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    torch.testing.assert_close(got.double(), ref, rtol=tol, atol=tol * big.double().abs().sum(1).max().item() * 1e-3)


@pytest.mark.gpu
def test_full_reduction_and_integers_and_unsplit_shapes():
    from torch_mojo_backend import eager_kernels as ek

    g = torch.Generator().manual_seed(1)
    flat = torch.randn(1, 8_000_011, generator=g).cuda()
    got, want, need = _both(flat, ek.SUM, ek)
    assert need > 0 and torch.equal(got.view(torch.int32), want.view(torch.int32))
    ints = torch.randint(-1000, 1000, (2, 300_000), generator=g, dtype=torch.int64).cuda()
    got, want, _ = _both(ints, ek.SUM, ek)
    assert torch.equal(got, want) and torch.equal(got.cpu(), ints.cpu().sum(1))
    got, want, _ = _both(ints, ek.AMAX, ek)
    assert torch.equal(got, want) and torch.equal(got.cpu(), ints.cpu().amax(1))
    rowsy = torch.randn(5000, 257, generator=g).cuda()                   # one pass, no scratch at all
    got, want, need = _both(rowsy, ek.AMAX, ek)
    assert need == 0 and torch.equal(got, want)


def test_limit_and_argument_errors_are_reported_before_any_launch():
    from torch_mojo_backend import eager_kernels as ek

    L = ek.lib()
    # 4000 rows x 3 partials x 16 bytes stays below the limit; a shape needing 2^30-element chunks
    # times thousands of rows would not: the plan is a pure function of the shape, so ask it.
    rows, cols = 4000, (1 << 30) * 6
    assert L.tmb_reduce_workspace_bytes(rows, cols, ek.F32) > STATIC_SCRATCH_BYTES
    assert L.tmb_reduce_rows_static(None, None, rows, cols, ek.SUM, ek.F32, None) == -4
    assert "static" in ek.status_string(-4)
    assert L.tmb_reduce_rows_static(None, None, -1, 4, ek.SUM, ek.F32, None) == -1
    assert L.tmb_reduce_rows_static(None, None, 1, 1 << 22, ek.SUM, ek.F32, None) == -1   # null pointers
    assert L.tmb_reduce_rows_static(None, None, 0, 4, ek.SUM, ek.F32, None) == 0
