"""The C-ABI library: it loads without a GPU, exports every symbol include/tmb_hip.h declares,
and rejects malformed arguments on the host before anything would be enqueued."""

import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tmb_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tmb_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from torch_mojo_backend import eager_kernels as ek

    declared = _declared_symbols()
    assert len(declared) >= 10
    handle = ctypes.CDLL(ek.LIBRARY_PATH)
    for name in declared:
        assert hasattr(handle, name), f"{name} declared in tmb_hip.h but not exported"
    assert sorted(ek.SIGNATURES) == declared, "ctypes signature table out of sync with the header"


def test_version_and_status_strings():
    from torch_mojo_backend import eager_kernels as ek

    L = ek.lib()
    assert L.tmb_version() == 1000
    assert ek.status_string(0) == "ok"
    assert "invalid" in ek.status_string(-1)
    assert "unsupported" in ek.status_string(-2)
    assert "workspace" in ek.status_string(-3)


def test_host_side_argument_validation_needs_no_gpu():
    from torch_mojo_backend import eager_kernels as ek

    L = ek.lib()
    # negative sizes / null pointers / unknown enums are refused before any launch
    assert L.tmb_softmax_rows(None, None, -1, 4, ek.F32, ek.F32, 0, None) == -1
    assert L.tmb_softmax_rows(None, None, 3, 4, ek.F32, ek.F32, 0, None) == -1
    assert L.tmb_softmax_rows(None, None, 0, 4, ek.F32, ek.F32, 0, None) == 0   # empty: nothing to do
    assert L.tmb_layer_norm_rows(None, None, None, None, None, None, 2, 2, 1e-5, ek.F32, ek.F32, None) == -1
    assert L.tmb_layer_norm_rows(None, None, None, None, None, None, 2, 2, 1e-5, ek.BF16, ek.F32, None) == -2   # never widens
    assert L.tmb_layer_norm_rows(None, None, None, None, None, None, 2, 2, 1e-5, ek.F16, ek.BF16, None) == -2
    assert L.tmb_reduce_rows(None, None, 2, 2, 7, ek.F32, None, 0, None) == -1  # unknown op
    assert L.tmb_reduce_rows(None, None, 2, 0, ek.SUM, ek.F32, None, 0, None) == -1
    assert L.tmb_argmax_rows(None, None, 2, 0, ek.F32, None, 0, None) == -1
    assert L.tmb_gemm(None, None, None, None, 1, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, ek.F32, 0, None) == -1
    assert L.tmb_gemm(None, None, None, None, 1, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, ek.I64, 0, None) == -2
    assert L.tmb_gemm(None, None, None, None, 1, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, ek.F32, 9, None) == -1
    assert L.tmb_gemm(None, None, None, None, 0, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, ek.F32, 0, None) == 0
    assert L.tmb_gelu(None, None, -5, ek.F32, 1, None) == -1
    # the entry points added later obey the same rules
    assert L.tmb_softmax_rows_scaled(None, None, 2, 2, ek.F32, 1.0, 0, 0, None) == -1
    strides = (ctypes.c_int64 * 3)(64, 64, 64)
    assert L.tmb_attention_fwd(None, None, None, None, None, 1, 1, 4, 4, 64, strides, strides, strides,
                               strides, 0.125, 0, 0, ek.BF16, None) == -1
    eight = [strides] * 8
    assert L.tmb_attention_bwd(*[None] * 10, 1, 1, 4, 4, 64, *eight, 0.125, 1, ek.BF16, None) == -1
    assert L.tmb_attention_bwd(*[None] * 10, 1, 1, 4, 4, 128, *eight, 0.125, 1, ek.BF16, None) == -2
    assert L.tmb_attention_bwd(*[None] * 10, 1, 1, 4, 4, 64, *eight, 0.125, 1, ek.F32, None) == -2
    assert L.tmb_attention_bwd(*[None] * 10, 0, 1, 4, 4, 64, *eight, 0.125, 1, ek.BF16, None) == 0
    assert L.tmb_attention_bwd_workspace_bytes(2, 3, 5) == 2 * 2 * 3 * 5 * 4
    assert L.tmb_gemm_residual(None, None, None, None, None, 1, 2, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, 0,
                               ek.BF16, ek.BF16, ek.BF16, 0, None) == -1
    # epilogue flags: only the rounding flag may be or-ed in; the float32 stream excludes it
    assert L.tmb_gemm(None, None, None, None, 1, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, ek.F32, 0x200, None) == -1
    assert L.tmb_gemm(None, None, None, None, 0, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, ek.F32,
                      ek.EPI_GELU_TANH | ek.EPI_ROUND_LIKE_UNFUSED, None) == 0
    assert L.tmb_gemm_residual(None, None, None, None, None, 1, 2, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, 0,
                               ek.BF16, ek.F16, ek.BF16, 0, None) == -1   # NULL residual comes first
    fake = ctypes.c_void_p(4096)   # never dereferenced: rejected on the host
    assert L.tmb_gemm_residual(fake, fake, fake, None, fake, 1, 2, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, 0,
                               ek.BF16, ek.F16, ek.BF16, 0, None) == -2   # residual type: T or fp32
    assert L.tmb_gemm_residual(fake, fake, fake, None, fake, 1, 2, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, 0,
                               ek.F32, ek.F32, ek.F32, 0, None) == -2     # fp32 A/B: caller adds separately
    assert L.tmb_gemm_ws(None, None, None, None, 1, 2, 2, 2, 2, 2, 2, 0, 0, 0, 0, 0, ek.F32, 0, None, 0,
                         None) == -1
    assert L.tmb_gelu_backward(None, None, None, 8, ek.F32, 0, None) == -1
    assert L.tmb_gelu_backward(None, None, None, 0, ek.F32, 0, None) == 0
    assert L.tmb_softmax_backward_rows(None, None, None, 2, 2, ek.F32, 0, None) == -1
    assert L.tmb_softmax_backward_rows(None, None, None, -2, 2, ek.F32, 0, None) == -1
    assert L.tmb_layer_norm_backward_rows(None, None, None, None, None, None, None, None, 2, 2,
                                          ek.F32, None, 0, None) == -1
    assert L.tmb_layer_norm_backward_rows(None, None, None, None, None, None, None, None, 2, 0,
                                          ek.F32, None, 0, None) == -1


def test_workspace_plan_is_a_pure_function_of_the_shape():
    from torch_mojo_backend import eager_kernels as ek

    L = ek.lib()
    assert L.tmb_reduce_workspace_bytes(65536, 4096, ek.F32) == 0        # one pass, no scratch
    full = L.tmb_reduce_workspace_bytes(1, 65536 * 4096, ek.F32)
    assert full > 0 and full % 16 == 0
    assert full == L.tmb_reduce_workspace_bytes(1, 65536 * 4096, ek.BF16)
    assert L.tmb_reduce_workspace_bytes(512, 50257, ek.F32) == 512 * 3 * 16
    assert L.tmb_reduce_workspace_bytes(0, 10, ek.F32) == 0
    # split-K scratch: only for half-precision products with fewer tiles than CUs and a long K
    assert L.tmb_gemm_workspace_bytes(1, 8192, 8192, 8192, ek.BF16) == 0
    assert L.tmb_gemm_workspace_bytes(1, 1024, 768, 3072, ek.F32) == 8 * 1024 * 768 * 4
    assert L.tmb_gemm_workspace_bytes(1, 4096, 4096, 4096, ek.F32) == 0
    assert L.tmb_gemm_workspace_bytes(1, 1024, 768, 3072, ek.BF16) == 5 * 1024 * 768 * 4
    assert L.tmb_gemm_workspace_bytes(2, 1024, 768, 3072, ek.BF16) == 0
    # layer-norm backward partials: a whole number of fp32 row pairs, same for both 16-bit types
    ln = L.tmb_layer_norm_backward_workspace_bytes(32768, 768, ek.BF16)
    assert ln > 0 and ln % (2 * 768 * 4) == 0
    assert ln == L.tmb_layer_norm_backward_workspace_bytes(32768, 768, ek.F16)
    assert L.tmb_layer_norm_backward_workspace_bytes(0, 768, ek.F32) == 0


def test_product_refuses_cpu_tensors_and_never_falls_back():
    from torch_mojo_backend.eager_kernels import hip_ops

    x = torch.randn(4, 8)
    for call in (lambda: hip_ops.softmax(x, -1), lambda: hip_ops.gemm(x, x.t()),
                 lambda: hip_ops.layer_norm(x, [8], None, None, 1e-5),
                 lambda: hip_ops.reduce(x, [1], False, 0), lambda: hip_ops.argmax(x, 1, False),
                 lambda: hip_ops.gelu(x)):
        with pytest.raises(TypeError, match="no CPU path"):
            call()


def test_missing_library_raises(monkeypatch, tmp_path):
    from torch_mojo_backend import eager_kernels as ek

    monkeypatch.setattr(ek, "_lib", None)
    monkeypatch.setattr(ek, "LIBRARY_PATH", str(tmp_path / "libtmb_hip.so"))
    with pytest.raises(ek.HipLibraryMissing, match="no CPU or PyTorch fallback"):
        ek.lib()


def test_library_path_can_name_another_build(tmp_path):
    """TORCH_MOJO_BACKEND_HIP_LIBRARY points the loader at another build of the library (a
    diagnostic variant); a path that does not exist fails as loudly as the default one."""
    import subprocess
    import sys

    bogus = str(tmp_path / "libtmb_hip_diag9.so")
    code = ("import sys; sys.path.insert(0, %r)\n"
            "from torch_mojo_backend import eager_kernels as ek\n"
            "assert ek.LIBRARY_PATH == %r, ek.LIBRARY_PATH\n"
            "try:\n    ek.lib()\nexcept ek.HipLibraryMissing as e:\n    print('missing:', e)\n"
            % (os.path.join(ROOT, "torch-max-backend_amd"), bogus))
    env = dict(os.environ, TORCH_MOJO_BACKEND_HIP_LIBRARY=bogus)
    done = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    assert "missing:" in done.stdout and "libtmb_hip_diag9.so" in done.stdout


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "torch-max-backend_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".sh")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(import|from)\s+oracle\b", text, flags=re.M), f
                assert "libtmb_oracle" not in text, f


def test_relayout_rules_on_the_host():
    """Pure host logic (no GPU): which layouts are re-laid, and into what."""
    from torch_mojo_backend.eager_kernels import hip_ops

    def prep(a, b):
        la, lb = hip_ops._matrix_layout(a), hip_ops._matrix_layout(b)
        m, k, n = a.shape[-2], a.shape[-1], b.shape[-1]
        ok = hip_ops._mfma_layouts_ok(a, b, la, lb, m, n, k, a.dim() == 3)
        return ok, (None if ok else hip_ops._relayout_for_mfma(a, b, la, lb, m, n, k, a.dim() == 3))

    bf = torch.bfloat16
    ok, _ = prep(torch.zeros(64, 256, dtype=bf), torch.zeros(256, 128, dtype=bf))
    assert ok
    # an odd contraction length (a vocabulary as K): both operands padded with zeros to 64 | K
    a, b = torch.randn(16, 1001).to(bf), torch.randn(1001, 24).to(bf)
    ok, (a2, b2, la, lb, k, rows) = prep(a, b)
    assert not ok and k == 1024 and rows == 16 and tuple(a2.shape) == (16, 1024) and tuple(b2.shape) == (1024, 24)
    assert la == (0, 1024) and lb == (0, 24)
    assert torch.equal(a2[:, :1001], a) and not a2[:, 1001:].any() and not b2[1001:].any()
    assert hip_ops._mfma_layouts_ok(a2, b2, la, lb, 16, 24, k, False)
    # the weight-gradient form with an odd M keeps its form: the stored [K, M] rows get zero
    # columns up to 64 | M (the width an odd contraction length gets, so that one padded copy can
    # serve both), B stays, and the launch computes the few extra rows
    a, b = torch.randn(512, 1001).to(bf).t(), torch.randn(512, 96).to(bf)
    ok, (a2, b2, la, lb, k, rows) = prep(a, b)
    assert not ok and rows == 1024 and la == (1, 1024) and tuple(a2.shape) == (1024, 512) and b2 is b
    assert torch.equal(a2[:1001], a) and not a2[1001:].any() and k == 512
    assert hip_ops._mfma_layouts_ok(a2, b2, la, lb, rows, 96, k, False)
    # ... but not with 64 or fewer columns (no weight-gradient kernel there): row-major A
    ok, (a2, b2, la, lb, k, rows) = prep(torch.randn(512, 1001).to(bf).t(), torch.randn(512, 64).to(bf))
    assert not ok and la == (0, 512) and rows == 1001
    # ... and the same form when it is eligible is left alone
    ok, _ = prep(torch.randn(512, 1024).to(bf).t(), torch.randn(512, 96).to(bf))
    assert ok
    # a narrow product behind a transposed A (attention's dV = P^T dO)
    ok, (a2, b2, la, lb, k, rows) = prep(torch.randn(3, 256, 128).to(bf).transpose(1, 2), torch.randn(3, 256, 64).to(bf))
    assert not ok and la == (0, 256) and b2.shape == (3, 256, 64) and rows == 128
    # N-major B with an odd pitch becomes K-major; float32 counts in vectors of four
    a, b = torch.randn(32, 64).to(bf), torch.randn(64, 77).to(bf)
    ok, (a2, b2, la, lb, k, rows) = prep(a, b)
    assert not ok and lb == (1, 64) and torch.equal(b2, b)
    ok, _ = prep(torch.zeros(8, 36), torch.zeros(36, 20))
    assert ok
    ok, (a2, b2, la, lb, k, rows) = prep(torch.randn(8, 50), torch.randn(50, 20))
    assert not ok and k == 64 and la == (0, 64)
