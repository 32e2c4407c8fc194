"""The committed fixtures (tests/golden/hot_ops_torch_cpu.npz: seeded inputs with PyTorch CPU
eager's outputs, written by tests/golden/make_fixtures.py) fed straight to the HIP kernels.

PyTorch CPU eager is what the reference's own tests compare every hot op with
(torch_mojo_backend/testing.py:186-229). These tests tie the kernels to those vectors without
the C restatement in between; tolerances are the ones of helpers.py (fixture outputs are
themselves rounded to their storage type, hence ``rounded_want``)."""

import os

import numpy as np
import pytest
import torch

from helpers import as64, assert_close64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def golden():
    path = os.path.join(os.path.dirname(__file__), "golden", "hot_ops_torch_cpu.npz")
    return np.load(path, allow_pickle=False)


def _t(arr, bf16=False):
    t = torch.from_numpy(np.ascontiguousarray(arr))
    return (t.view(torch.bfloat16) if bf16 else t).to("cuda")


def _ops():
    from torch_mojo_backend.eager_kernels import hip_ops
    return hip_ops


@pytest.mark.parametrize("log", [False, True])
def test_softmax_fixture(golden, log):
    x = _t(golden["softmax_x"])
    want = golden["log_softmax_y" if log else "softmax_y"]
    got = _ops().softmax(x, -1, log=log)
    assert_close64(got, want.astype(np.float64), rounded_want=True, what="softmax fixture")


def test_softmax_fixture_through_the_registry(golden):
    from torch_mojo_backend.aten_functions import MAPPING_TORCH_ATEN_TO_MOJO as mapping
    aten = torch.ops.aten
    x = _t(golden["softmax_x"])
    got = mapping[aten._softmax](x, -1, False)
    assert_close64(got, golden["softmax_y"].astype(np.float64), rounded_want=True, what="_softmax")
    got = mapping[aten._log_softmax](x, -1, False)
    assert_close64(got, golden["log_softmax_y"].astype(np.float64), rounded_want=True,
                   what="_log_softmax")


def test_layer_norm_fixture(golden):
    x, w, b = (_t(golden[k], bf16=True) for k in ("ln_x", "ln_w", "ln_b"))
    out, mean, rstd = _ops().layer_norm(x, [65], w, b, 1e-5)
    assert out.dtype == torch.bfloat16
    want = as64(_t(golden["ln_out"], bf16=True))
    assert_close64(out, want, rounded_want=True, what="layer norm fixture")
    # PyTorch stores bf16 statistics for bf16 input; the fixture holds them widened again
    assert_close64(mean.float().reshape(-1), golden["ln_mean"].astype(np.float64).reshape(-1),
                   rtol=2.0 ** -7, atol=2.0 ** -7, what="mean")
    assert_close64(rstd.float().reshape(-1), golden["ln_rstd"].astype(np.float64).reshape(-1),
                   rtol=2.0 ** -7, atol=2.0 ** -7, what="rstd")


def test_argmax_fixture_is_exact(golden):
    x = _t(golden["argmax_x"])
    got = _ops().argmax(x, 1, False)
    assert got.dtype == torch.int64
    assert np.array_equal(got.cpu().numpy(), golden["argmax_y"])


def test_addmm_fixture(golden):
    a, b, bias = (_t(golden[k], bf16=True) for k in ("mm_a", "mm_b", "mm_bias"))
    got = _ops().gemm(a, b, bias)
    want = as64(_t(golden["mm_out"], bf16=True))
    assert_close64(got, want, rounded_want=True, what="addmm fixture")
    from torch_mojo_backend.aten_functions import MAPPING_TORCH_ATEN_TO_MOJO as mapping
    got = mapping[torch.ops.aten.addmm](bias, a, b)
    assert_close64(got, want, rounded_want=True, what="aten.addmm fixture")


def test_row_reduction_fixtures(golden):
    from torch_mojo_backend import eager_kernels as ek
    x = _t(golden["sum_x"])
    bound = (x.shape[1] - 1) * 2.0 ** -24 * as64(x.abs().sum(1))
    got = _ops().reduce(x, [1], False, ek.SUM)
    assert_close64(got, golden["sum_rows"].astype(np.float64), extra_abs=2 * bound, what="sum rows")
    got = _ops().reduce(x, [1], False, ek.AMAX)
    assert np.array_equal(got.cpu().numpy(), golden["amax_rows"])
