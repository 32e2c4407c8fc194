"""GPU parity of the GEMM family (mm / addmm / bmm / linear, bias + GELU epilogue)."""

import math

import numpy as np
import pytest
import torch

import oracle
from oracle import closed_form as cf
from helpers import as64, assert_close64, rel_frobenius, seeded

pytestmark = pytest.mark.gpu

HALF = [torch.bfloat16, torch.float16]


def _ops():
    from torch_mojo_backend.eager_kernels import hip_ops
    return hip_ops


def _ek():
    from torch_mojo_backend import eager_kernels
    return eager_kernels


def _dev(t):
    return t.to("cuda")


def _abc(m, n, k, dtype, seed=0):
    return (seeded((m, k), seed=seed, dtype=dtype), seeded((k, n), seed=seed + 1, dtype=dtype),
            seeded((n,), seed=seed + 2, dtype=dtype))


# Tiny cases: the C oracle (sequential fp32, the reference's _cpu_gemm_naive) is the yardstick.
TINY = [(1, 1, 8), (3, 5, 16), (33, 65, 72), (64, 64, 64), (129, 131, 200), (257, 96, 1000)]


@pytest.mark.parametrize("dtype", [torch.float32] + HALF)
@pytest.mark.parametrize("mnk", TINY)
@pytest.mark.parametrize("trans_b", [False, True])
def test_addmm_small_vs_c_oracle(mnk, dtype, trans_b):
    m, n, k = mnk
    a, b, bias = _abc(m, n, k, dtype)
    if trans_b:  # B given as the .t() view of an [n, k] weight
        b = b.t().contiguous().t()
    got = _ops().gemm(_dev(a), _dev(b), _dev(bias))
    assert got.dtype == dtype and tuple(got.shape) == (m, n)
    want = cf.gemm(as64(a), as64(b), as64(bias))
    # fp32 accumulation of k products of magnitude ~1: error <= k*2^-24*sum|a||b| a priori
    bound = k * 2.0 ** -24 * (np.abs(as64(a)) @ np.abs(as64(b)) + np.abs(as64(bias)))
    assert_close64(got, want, extra_abs=bound, what=f"addmm {mnk} {dtype}")
    ref = oracle.gemm(a, b, bias)
    assert_close64(got, as64(ref), extra_abs=2 * bound, rounded_want=True, what="vs C oracle")


# Benchmark GEMM shapes that the CPU can check in seconds + the reference's awkward shapes
# (N=50257 / 3001 unaligned, K=1000, M=257).
MID = [(128, 768, 768), (1024, 3072, 768), (1024, 768, 3072), (512, 2304, 768), (257, 3001, 1000),
       (512, 50257, 768), (300, 260, 264)]


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("mnk", MID)
@pytest.mark.parametrize("trans_b", [False, True])
def test_addmm_half_frobenius(mnk, dtype, trans_b):
    m, n, k = mnk
    a, b, bias = _abc(m, n, k, dtype, seed=3)
    if trans_b:
        b = b.t().contiguous().t()
    got = _ops().gemm(_dev(a), _dev(b), _dev(bias))
    want = (a.float() @ b.float() + bias.float()).double().numpy()
    assert rel_frobenius(got, want) <= 1e-2
    # elementwise: one storage ulp of the exact value plus fp32 accumulation slack
    assert_close64(got, want, rtol=2e-5, atol=1e-3, what=f"addmm {mnk} {dtype}")


@pytest.mark.parametrize("mnk", [(128, 768, 768), (1024, 3072, 768), (130, 50257, 768)])
def test_mm_fp32(mnk):
    m, n, k = mnk
    a, b, _ = _abc(m, n, k, torch.float32, seed=5)
    got = _ops().gemm(_dev(a), _dev(b.t().contiguous().t()))
    want = a.double().numpy() @ b.double().numpy()
    bound = k * 2.0 ** -24 * (np.abs(as64(a)) @ np.abs(as64(b)))
    assert_close64(got, want, extra_abs=bound, what=f"mm fp32 {mnk}")


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("mnk", [(4096, 4096, 4096), (7000, 7096, 4096), (4000, 4104, 4096),
                                 (2100, 3000, 768),
                                 # 32-deep stages as single k-steps: alternating fragment slots with an
                                 # odd and an even number of steps, and the one-slot configuration
                                 (2048, 4096, 2048), (2048, 4096, 1056), (2000, 4104, 1056),
                                 (5000, 9000, 1024),
                                 # one partial round of 256 x 256 tiles; 256 x 128 tiles with 32-deep
                                 # stages (K-major B, K an odd multiple of 32)
                                 (3000, 3400, 2048), (3000, 3400, 8192), (16500, 1000, 992)])
@pytest.mark.parametrize("trans_b", [False, True])
def test_addmm_half_long_k_ragged_tiles(mnk, dtype, trans_b):
    """Products that run on the ring configurations with the 16x16x32 MFMA (256x256x64, 256x128x64,
    128x128x32 with K-major B, 128x256x32 with N-major B) and on their 32x32x16 neighbours in the
    tile choice, in both storage types, with whole and with ragged edge tiles: rows sampled from the first, the last and the interior tiles against
    float64, every column."""
    m, n, k = mnk
    g = torch.Generator(device="cuda").manual_seed(7)
    a = torch.randn(m, k, generator=g, device="cuda").to(dtype)
    b = torch.randn(k, n, generator=g, device="cuda").to(dtype)
    if trans_b:
        b = b.t().contiguous().t()
    bias = torch.randn(n, generator=g, device="cuda").to(dtype)
    got = _ops().gemm(a, b, bias)
    rows = torch.cat([torch.arange(0, 40), torch.arange(m - 40, m),
                      torch.randperm(m, generator=torch.Generator().manual_seed(2))[:48]]).to("cuda")
    want = (a[rows].cpu().double() @ b.cpu().double() + bias.cpu().double()).numpy()
    assert rel_frobenius(got[rows], want) <= 1e-2
    assert_close64(got[rows], want, rtol=2e-5, atol=2e-3, what=f"rows of {mnk} {dtype}")
    assert torch.equal(got, _ops().gemm(a, b, bias))


@pytest.mark.parametrize("mnk", [(4096, 4096, 4096), (8192, 8192, 8192)])
@pytest.mark.parametrize("trans_b", [False, True])
def test_addmm_bf16_large_sampled_rows(mnk, trans_b):
    """Benchmark sizes: float64 check on 64 sampled rows + linearity over the whole product."""
    m, n, k = mnk
    g = torch.Generator(device="cuda").manual_seed(0)
    a = torch.randn(m, k, generator=g, device="cuda").bfloat16()
    b = torch.randn(k, n, generator=g, device="cuda").bfloat16()
    if trans_b:
        b = b.t().contiguous().t()
    bias = torch.randn(n, generator=g, device="cuda").bfloat16()
    got = _ops().gemm(a, b, bias)
    rows = torch.randperm(m, generator=torch.Generator().manual_seed(1))[:64]
    a_s = a[rows.to("cuda")].cpu().double()
    want = (a_s @ b.cpu().double() + bias.cpu().double()).numpy()
    assert rel_frobenius(got[rows.to("cuda")], want) <= 1e-2
    assert_close64(got[rows.to("cuda")], want, rtol=2e-5, atol=2e-3, what=f"rows of {mnk}")
    # (2A)B + bias - bias == 2(AB) exactly in every rounding step => compare against no-bias runs
    c1 = _ops().gemm(a, b)
    c2 = _ops().gemm(a * 2, b)
    assert torch.equal(c2, c1 * 2)
    # determinism
    assert torch.equal(got, _ops().gemm(a, b, bias))


@pytest.mark.parametrize("dtype", [torch.float32] + HALF)
def test_bmm(dtype):
    a = seeded((12, 128, 64), seed=1, dtype=dtype)
    b = seeded((12, 128, 64), seed=2, dtype=dtype)
    v = seeded((12, 128, 64), seed=3, dtype=dtype)
    scores = _ops().gemm(_dev(a), _dev(b).transpose(1, 2))        # q @ k^T   (K-major B)
    want = torch.bmm(a.double(), b.double().transpose(1, 2)).numpy()
    assert_close64(scores, want, rtol=2e-5, atol=1e-4, what="q@k^T")
    ctx = _ops().gemm(_dev(seeded((12, 128, 128), seed=4, dtype=dtype)), _dev(v))  # att @ v (N-major B)
    want2 = torch.bmm(seeded((12, 128, 128), seed=4, dtype=dtype).double(), v.double()).numpy()
    assert_close64(ctx, want2, rtol=2e-5, atol=1e-4, what="att@v")
    ref = oracle.gemm(a, b.transpose(1, 2))
    assert_close64(scores, as64(ref), rtol=2e-5, atol=1e-4, rounded_want=True, what="vs C oracle")


# K >= 256 takes the direct-to-LDS ring kernel; the shapes are chosen so that each of its tile
# configurations runs, with ragged M and N edges: 256x256 with 64-deep stages (256 tiles = one
# round of the 256 CUs; K = 320 is five stages), 256x128 (528 tiles), 128x128 with 32-deep stages
# (K = 352 is not a multiple of 64), the short-K rings that run two workgroups per CU (256x128x32
# for K-major B at (8000, 2200, 352); 128x256x32 for the N-major twins of the large shapes), and
# shapes that stay on the register-staged kernel (few tiles, K < 256).
KMAJOR = [(3900, 4000, 320), (4000, 4100, 256), (4000, 4104, 448), (600, 1000, 352),
          (8000, 2200, 352), (1000, 5000, 128), (130, 70, 1152)]


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("mnk", KMAJOR)
def test_addmm_kmajor_b_tiles(mnk, dtype):
    m, n, k = mnk
    g = torch.Generator(device="cuda").manual_seed(11)
    a = torch.randn(m, k, generator=g, device="cuda").to(dtype)
    w = torch.randn(n, k, generator=g, device="cuda").to(dtype)      # weight [n, k]; B = w.t()
    bias = torch.randn(n, generator=g, device="cuda").to(dtype)
    got = _ops().gemm(a, w.t(), bias)
    want = (a.double() @ w.double().t() + bias.double()).cpu().numpy()
    assert rel_frobenius(got, want) <= 1e-2
    assert_close64(got, want, rtol=2e-5, atol=1e-3, what=f"addmm K-major B {mnk} {dtype}")
    # same product through the N-major path (other kernel, same fp32 accumulation order per
    # output is not guaranteed, so compare to the same bound rather than bit-for-bit)
    got_nn = _ops().gemm(a, w.t().contiguous(), bias)
    assert_close64(got_nn, want, rtol=2e-5, atol=1e-3, what=f"addmm N-major B {mnk} {dtype}")


def test_bmm_kmajor_b_direct_to_lds():
    a = seeded((12, 300, 256), seed=1, dtype=torch.bfloat16)
    b = seeded((12, 200, 256), seed=2, dtype=torch.bfloat16)
    got = _ops().gemm(_dev(a), _dev(b).transpose(1, 2))
    want = torch.bmm(a.double(), b.double().transpose(1, 2)).numpy()
    assert_close64(got, want, rtol=2e-5, atol=1e-4, what="bmm K-major B, K=256")
    assert_close64(got, as64(oracle.gemm(a, b.transpose(1, 2))), rtol=2e-5, atol=1e-4,
                   rounded_want=True, what="vs C oracle")


def test_bmm_benchmark_shape_bf16():
    a = seeded((48, 1024, 64), seed=1, dtype=torch.bfloat16)
    b = seeded((48, 64, 1024), seed=2, dtype=torch.bfloat16)
    got = _ops().gemm(_dev(a), _dev(b))
    want = torch.bmm(a.float(), b.float()).double().numpy()
    assert rel_frobenius(got, want) <= 1e-2
    assert_close64(got, want, rtol=2e-5, atol=1e-4, what="bmm [48,1024,64]x[48,64,1024]")


@pytest.mark.parametrize("dtype", [torch.float32] + HALF)
@pytest.mark.parametrize("approximate", ["tanh", "none"])
@pytest.mark.parametrize("trans_b", [False, True])
def test_gelu_epilogue_equals_unfused(dtype, approximate, trans_b):
    """round_like_unfused: bit-identical to addmm followed by the standalone GELU. Default: the
    GELU of the float32 sum, one cast - within one rounding of the float64 closed form."""
    m, n, k = 200, 3072, 768
    a, b, bias = _abc(m, n, k, dtype, seed=9)
    b = (b * 0.05).to(dtype)
    if trans_b:
        b = b.t().contiguous().t()
    ek = _ek()
    epi = ek.EPI_GELU_TANH if approximate == "tanh" else ek.EPI_GELU_ERF
    fused = _ops().gemm(_dev(a), _dev(b), _dev(bias), epilogue=epi, round_like_unfused=True)
    unfused = _ops().gelu(_ops().gemm(_dev(a), _dev(b), _dev(bias)), approximate)
    assert torch.equal(fused, unfused)
    pre = (a.double() @ b.double() + bias.double()).numpy()
    want = cf.gelu_tanh(pre) if approximate == "tanh" else cf.gelu_erf(pre)
    assert_close64(fused, want, rtol=2e-2 if dtype != torch.float32 else 1e-4, atol=2e-3,
                   what="gelu epilogue vs closed form")
    # one cast: the float32 accumulation error (k products of magnitude ~0.05) goes through a
    # function of slope <= 1.13, then half a unit of the storage type
    once = _ops().gemm(_dev(a), _dev(b), _dev(bias), epilogue=epi)
    acc_err = 1.13 * k * 2.0 ** -24 * (a.double().abs() @ b.double().abs()).numpy()
    assert_close64(once, want, rtol=1e-5, atol=1e-6, extra_abs=acc_err, what="gelu of the fp32 sum")
    if dtype == torch.float32:
        assert torch.equal(once, fused)          # nothing to round in between


@pytest.mark.parametrize("dtype", [torch.float32] + HALF)
@pytest.mark.parametrize("approximate", ["tanh", "none"])
def test_gelu_standalone(dtype, approximate):
    x = seeded((1000, 129), seed=2, scale=3.0, dtype=dtype)
    got = _ops().gelu(_dev(x), approximate)
    want = cf.gelu_tanh(as64(x)) if approximate == "tanh" else cf.gelu_erf(as64(x))
    assert_close64(got, want, rtol=1e-5, atol=2e-6, what="gelu")
    assert_close64(got, as64(oracle.gelu(x, approximate)), rtol=1e-5, atol=2e-6, rounded_want=True, what="vs C oracle")


def test_bias_is_added_before_the_cast():
    """acc + bias is rounded once. acc = 1 + 2^-8 is a bf16 tie that rounds to 1.0 on its own;
    with bias 2^-10 the fp32 sum lies above the tie and must round UP to 1 + 2^-7, whereas
    round(acc) + bias would give 1.0."""
    k = 8
    a = torch.zeros(1, k, dtype=torch.bfloat16)
    b = torch.zeros(k, 1, dtype=torch.bfloat16)
    a[0, 0], b[0, 0] = 1.0, 1.0
    a[0, 1], b[1, 0] = 2.0 ** -8, 1.0
    bias = torch.tensor([2.0 ** -10], dtype=torch.bfloat16)
    want = torch.tensor([[1.0 + 2.0 ** -7]]).bfloat16()
    assert torch.equal(oracle.gemm(a, b, bias), want)
    assert torch.equal(_ops().gemm(_dev(a), _dev(b), _dev(bias)).cpu(), want)
    # same thing through the MFMA path (needs k % 8 == 0, which k = 8 satisfies) and the SIMT
    # path (fp32 storage keeps every bit, so only check it runs and is exact)
    got32 = _ops().gemm(_dev(a.float()), _dev(b.float()), _dev(bias.float())).cpu()
    assert got32.item() == 1.0 + 2.0 ** -8 + 2.0 ** -10


def test_degenerate_shapes():
    ops = _ops()
    a = _dev(seeded((0, 16), dtype=torch.float32))
    b = _dev(seeded((16, 8), dtype=torch.float32))
    assert ops.gemm(a, b).shape == (0, 8)
    a2 = _dev(seeded((4, 0), dtype=torch.float32))
    b2 = _dev(seeded((0, 8), dtype=torch.float32))
    bias = _dev(seeded((8,), dtype=torch.float32))
    assert torch.equal(ops.gemm(a2, b2), torch.zeros(4, 8, device="cuda"))
    assert torch.equal(ops.gemm(a2, b2, bias), bias.expand(4, 8))
    one = ops.gemm(_dev(seeded((1, 768), seed=1)), _dev(seeded((768, 1), seed=2)))
    assert one.shape == (1, 1)


def test_gemm_rejects_cpu_tensors():
    with pytest.raises(TypeError, match="no CPU path"):
        _ops().gemm(torch.randn(2, 2), torch.randn(2, 2))


def test_queued_launches_are_bit_identical():
    a, b, bias = _abc(512, 768, 768, torch.bfloat16, seed=4)
    ad, bd, cd = _dev(a), _dev(b), _dev(bias)
    outs = [_ops().gemm(ad, bd, cd) for _ in range(3)]
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])


# residual added in the GEMM's own epilogue. With round_like_unfused it must give the bits of
# gemm(...) + residual; by default the sum is formed in float32 and cast once, and residual and
# result may be float32 next to 16-bit operands. Shapes cover the ring configurations (see
# KMAJOR), the register-staged kernel (K = 128) and an odd row pitch; float32 operands have no
# fused path and take the separate add inside the same call.
RESIDUAL = [(3900, 4000, 320), (4000, 4104, 448), (600, 1000, 352), (8000, 2200, 352),
            (1000, 5000, 128), (512, 50257, 768), (32768, 768, 768)]


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("mnk", RESIDUAL)
@pytest.mark.parametrize("trans_b", [False, True])
def test_residual_epilogue_equals_separate_add(mnk, dtype, trans_b):
    m, n, k = mnk
    g = torch.Generator(device="cuda").manual_seed(21)
    a = torch.randn(m, k, generator=g, device="cuda").to(dtype)
    b = (torch.randn(n, k, generator=g, device="cuda") * 0.1).to(dtype)
    b = b.t() if trans_b else b.t().contiguous()
    bias = torch.randn(n, generator=g, device="cuda").to(dtype)
    res = torch.randn(m, n, generator=g, device="cuda").to(dtype)
    fused = _ops().gemm(a, b, bias, residual=res, round_like_unfused=True)
    plain = _ops().gemm(a, b, bias) + res
    assert torch.equal(fused, plain)


def _residual_reference(a, b, bias, rows):
    """float64 a[rows] @ b + bias on the device, plus the fp32 accumulation bound."""
    a64, b64 = a[rows].double(), b.double()
    exact = a64 @ b64 + bias.double()
    bound = a.shape[1] * 2.0 ** -24 * (a64.abs() @ b64.abs())
    return exact, bound


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("mnk", RESIDUAL)
@pytest.mark.parametrize("resid_f32,out_f32", [(False, False), (True, True), (True, False), (False, True)])
def test_residual_epilogue_in_float32_one_cast(mnk, dtype, resid_f32, out_f32):
    """Default mode: c = OUT(acc + bias + residual), everything in float32 up to the one cast;
    residual and result in the operands' type or float32. Checked on sampled rows against
    float64 (the accumulation bound plus half a unit of the output type)."""
    m, n, k = mnk
    g = torch.Generator(device="cuda").manual_seed(23)
    a = torch.randn(m, k, generator=g, device="cuda").to(dtype)
    b = (torch.randn(n, k, generator=g, device="cuda") * 0.1).to(dtype).t()
    bias = torch.randn(n, generator=g, device="cuda").to(dtype)
    res = torch.randn(m, n, generator=g, device="cuda") * 3
    res = res if resid_f32 else res.to(dtype)
    out = _ops().gemm(a, b, bias, residual=res, out_dtype=torch.float32 if out_f32 else None)
    assert out.dtype == (torch.float32 if out_f32 else dtype) and tuple(out.shape) == (m, n)
    rows = torch.tensor(sorted({0, 1, 31, 32, 127, 128, 255, 256, m // 2, m - 129, m - 2, m - 1}),
                        device="cuda")
    exact, bound = _residual_reference(a, b, bias, rows)
    want = (exact + res[rows].double()).cpu().numpy()
    assert_close64(out[rows], want, rtol=1e-6, atol=1e-6, extra_abs=bound.cpu().numpy(),
                   what=f"residual epilogue {mnk} resid_f32={resid_f32} out_f32={out_f32}")
    if not resid_f32 and not out_f32:
        # and it is closer to the truth than the unfused order, which rounds the product first
        twice = _ops().gemm(a, b, bias, residual=res, round_like_unfused=True)
        e_once = (out[rows].double() - torch.from_numpy(want).cuda()).abs().mean().item()
        e_twice = (twice[rows].double() - torch.from_numpy(want).cuda()).abs().mean().item()
        assert e_once <= e_twice


# A float32 residual stream over whole tiles, every element checked: the residual of a wave tile is
# requested as a whole before its bands are staged. Shapes: one tile per workgroup, two and three
# tiles per workgroup, short K, and (below) a batch.
STREAM_TILES = [(8192, 1024, 768), (16384, 768, 768), (32768, 768, 768), (16384, 768, 3072), (32768, 768, 192),
                (32768, 1536, 128), (65536, 256, 256)]


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("mnk", STREAM_TILES)
def test_float32_residual_stream_over_whole_tiles(mnk, dtype):
    m, n, k = mnk
    g = torch.Generator(device="cuda").manual_seed(29)
    a = torch.randn(m, k, generator=g, device="cuda").to(dtype)
    w = (torch.randn(n, k, generator=g, device="cuda") * 0.1).to(dtype)
    bias = torch.randn(n, generator=g, device="cuda").to(dtype)
    res = torch.randn(m, n, generator=g, device="cuda") * 3
    out = _ops().gemm(a, w.t(), bias, residual=res, out_dtype=torch.float32)
    # every element, against float64
    exact = a.double() @ w.double().t() + bias.double()
    bound = k * 2.0 ** -24 * (a.double().abs() @ w.double().abs().t())
    err = (out.double() - (exact + res.double())).abs()
    limit = bound + 1e-6 + 1e-6 * (exact + res.double()).abs()
    worst = (err - limit).max().item()
    assert worst <= 0, f"{mnk} {dtype}: {worst} over the bound at {torch.nonzero(err > limit)[:4].tolist()}"
    # and the same bits for a residual whose rows do not start on 16-byte boundaries
    wide = torch.zeros(m, n + 1, device="cuda")
    wide[:, :n] = res
    assert torch.equal(out, _ops().gemm(a, w.t(), bias, residual=wide[:, :n], out_dtype=torch.float32))
    # again into a used buffer: nothing of an earlier launch may survive
    again = _ops().gemm(a, w.t(), bias, residual=res, out_dtype=torch.float32)
    assert torch.equal(out, again)


def test_float32_residual_stream_batched():
    g = torch.Generator(device="cuda").manual_seed(30)
    a = torch.randn(3, 8192, 320, generator=g, device="cuda").bfloat16()
    b = (torch.randn(3, 384, 320, generator=g, device="cuda") * 0.1).bfloat16()
    res = torch.randn(3, 8192, 384, generator=g, device="cuda")
    out = _ops().gemm(a, b.transpose(1, 2), residual=res, out_dtype=torch.float32)
    want = torch.bmm(a.double(), b.double().transpose(1, 2)) + res.double()
    torch.testing.assert_close(out.double(), want, rtol=1e-5, atol=1e-4)


# A product without bias whose output streams to memory (256 MB and more) runs persistent
# workgroups that request the next tile's operands before they store the finished one. Whole
# tiles only, tiles cut by both edges, and a row count that leaves some workgroups a tile short.
@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("mnk", [(8192, 16384, 768), (8192, 50257, 768), (8100, 16648, 320), (16384, 8192, 128)])
def test_streamed_product_without_bias(mnk, dtype):
    m, n, k = mnk
    g = torch.Generator(device="cuda").manual_seed(31)
    a = torch.randn(m, k, generator=g, device="cuda").to(dtype)
    w = (torch.randn(n, k, generator=g, device="cuda") * 0.1).to(dtype)
    out = _ops().gemm(a, w.t())
    assert tuple(out.shape) == (m, n) and out.dtype == dtype
    for lo in range(0, m, 2048):  # every element, in slabs of rows
        hi = min(m, lo + 2048)
        exact = a[lo:hi].double() @ w.double().t()
        bound = k * 2.0 ** -24 * (a[lo:hi].double().abs() @ w.double().abs().t())
        err = (out[lo:hi].double() - exact).abs()
        ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
        limit = bound + ulp * exact.abs() + 1e-6
        worst = (err - limit).max().item()
        assert worst <= 0, f"{mnk} {dtype} rows {lo}..{hi}: {worst} over the bound"
    assert torch.equal(out, _ops().gemm(a, w.t()))


def test_float32_stream_rejects_the_bit_identical_mode_and_composes_with_layer_norm():
    g = torch.Generator(device="cuda").manual_seed(24)
    a = torch.randn(512, 768, generator=g, device="cuda").bfloat16()
    w = (torch.randn(768, 768, generator=g, device="cuda") * 0.02).bfloat16()
    bias = torch.zeros(768, device="cuda").bfloat16()
    x32 = torch.randn(512, 768, generator=g, device="cuda")
    with pytest.raises(ValueError, match="round_like_unfused"):
        _ops().gemm(a, w.t(), bias, residual=x32, round_like_unfused=True)
    with pytest.raises(TypeError, match="residual only"):
        _ops().gemm(a, w.t(), bias, out_dtype=torch.float32)
    y32 = _ops().gemm(a, w.t(), bias, residual=x32, out_dtype=torch.float32)
    gamma = torch.ones(768, device="cuda").bfloat16()
    h, _, _ = _ops().layer_norm(y32, [768], gamma, bias, 1e-5, need_stats=False, out_dtype=torch.bfloat16)
    want = torch.nn.functional.layer_norm(a.double() @ w.double().t() + x32.double(), [768])
    assert h.dtype == torch.bfloat16
    torch.testing.assert_close(h.double(), want, rtol=2.0 ** -8, atol=2.0 ** -8)


def test_residual_with_gelu_batches_and_fallbacks():
    ek = _ek()
    g = torch.Generator(device="cuda").manual_seed(22)
    a = torch.randn(6, 300, 256, generator=g, device="cuda").bfloat16()
    b = (torch.randn(6, 256, 200, generator=g, device="cuda") * 0.1).bfloat16()
    res = torch.randn(6, 300, 200, generator=g, device="cuda").bfloat16()
    assert torch.equal(_ops().gemm(a, b, residual=res, round_like_unfused=True), _ops().gemm(a, b) + res)
    # batched, one cast, float32 residual and result
    got = _ops().gemm(a, b, residual=res.float(), out_dtype=torch.float32)
    want = torch.bmm(a.double(), b.double()) + res.double()
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-4)
    a2, b2, r2 = a[0], b[0], res[0]
    bias = torch.randn(200, generator=g, device="cuda").bfloat16()
    fused = _ops().gemm(a2, b2, bias, epilogue=ek.EPI_GELU_TANH, residual=r2, round_like_unfused=True)
    assert torch.equal(fused, _ops().gemm(a2, b2, bias, epilogue=ek.EPI_GELU_TANH,
                                          round_like_unfused=True) + r2)
    # GELU in front of a float32 add: no kernel, composed inside the same call, summed in float32
    both = _ops().gemm(a2, b2, bias, epilogue=ek.EPI_GELU_TANH, residual=r2)
    want = torch.nn.functional.gelu(a2.double() @ b2.double() + bias.double(), approximate="tanh") + r2.double()
    torch.testing.assert_close(both.double(), want, rtol=2.0 ** -7, atol=2.0 ** -7)
    # a residual that is a column slice of something wider (row pitch > n)
    wide = torch.randn(300, 512, generator=g, device="cuda").bfloat16()
    assert torch.equal(_ops().gemm(a2, b2, bias, residual=wide[:, 100:300], round_like_unfused=True),
                       _ops().gemm(a2, b2, bias) + wide[:, 100:300])
    # float32: no fused kernel, same call, same bits as the two ops
    a32, b32, r32 = a2.float(), b2.float(), r2.float()
    assert torch.equal(_ops().gemm(a32, b32, residual=r32), _ops().gemm(a32, b32) + r32)
    with pytest.raises(ValueError):
        _ops().gemm(a2, b2, residual=r2[:, :100])


# ---- transposed A (the weight-gradient product dy^T x) -------------------------------------------
# (m, n, k): A is the .t() view of a [k, m] matrix, B is [k, n]. The MFMA ring takes m, n multiples
# of 8 with k a multiple of 32 and >= 256 (both tile sizes are covered); the rest is the SIMT path.
TRANS_A = [(768, 768, 4096), (256, 264, 512), (264, 136, 320), (3072, 768, 2048), (520, 776, 256),
           (100, 72, 200)]


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("mnk", TRANS_A)
def test_mm_transposed_a(mnk, dtype):
    m, n, k = mnk
    a_km = seeded((k, m), seed=1, dtype=dtype)
    b = seeded((k, n), seed=2, dtype=dtype)
    got = _ops().gemm(_dev(a_km).t(), _dev(b))
    assert got.dtype == dtype and tuple(got.shape) == (m, n)
    want = as64(a_km).T @ as64(b)
    assert rel_frobenius(got, want) <= (1e-2 if dtype == torch.bfloat16 else 2e-3)
    # every element, not just the norm: fp32 accumulation + one rounding to the storage type
    ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    assert np.abs(as64(got) - want).max() <= ulp * np.abs(want).max() + 1e-3


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("mnk", [(16392, 768, 2048), (8200, 3072, 1024),
                                 # a last round of 256 x 256 tiles that would be mostly empty:
                                 # 128 x 256 tiles, even and odd numbers of 32-deep stages
                                 (24008, 768, 2048), (24008, 776, 1056)])
def test_mm_transposed_a_many_tiles(mnk, dtype):
    """Enough tiles for the unsplit rings with both operands staged k-outer (the vocabulary
    projection's weight gradient): sampled rows, every column, against float64; the last tile
    row is ragged."""
    m, n, k = mnk
    g = torch.Generator(device="cuda").manual_seed(11)
    a_km = torch.randn(k, m, generator=g, device="cuda").to(dtype)
    b = torch.randn(k, n, generator=g, device="cuda").to(dtype)
    got = _ops().gemm(a_km.t(), b)
    assert got.dtype == dtype and tuple(got.shape) == (m, n)
    rows = torch.cat([torch.arange(0, 33), torch.arange(m - 33, m),
                      torch.randperm(m, generator=torch.Generator().manual_seed(3))[:40]]).to("cuda")
    want = (a_km[:, rows].cpu().double().t() @ b.cpu().double()).numpy()
    assert rel_frobenius(got[rows], want) <= (1e-2 if dtype == torch.bfloat16 else 2e-3)
    ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    assert np.abs(as64(got[rows]) - want).max() <= ulp * np.abs(want).max() + 1e-3
    assert torch.equal(got, _ops().gemm(a_km.t(), b))


def test_mm_transposed_a_batched_and_strided():
    # a pitch wider than m, batches, and the result of the same product through the SIMT path
    k, m, n = 512, 256, 320
    a_store = seeded((3, k, m + 24), seed=3, dtype=torch.bfloat16)
    b = seeded((3, k, n), seed=4, dtype=torch.bfloat16)
    a_view = _dev(a_store)[:, :, :m].transpose(1, 2)
    got = _ops().gemm(a_view, _dev(b))
    want = np.einsum("bkm,bkn->bmn", as64(a_store)[:, :, :m], as64(b))
    assert rel_frobenius(got, want) <= 1e-2


# ---- split-K (few output tiles, long K) ----------------------------------------------------------
SPLITK = [  # (m, n, k, trans_a, trans_b)
    (1024, 768, 3072, False, False), (1024, 768, 3072, False, True), (128, 768, 4096, False, True),
    (3072, 768, 8192, True, False), (768, 768, 32768, True, False), (264, 136, 2048, False, False),
    (100, 72, 2304, False, True),
]


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("case", SPLITK)
def test_split_k_matches_float64_and_the_unsplit_kernel(case, dtype):
    m, n, k, ta, tb = case
    a = seeded((k, m) if ta else (m, k), seed=21, dtype=dtype) * 0.25
    b = seeded((n, k) if tb else (k, n), seed=22, dtype=dtype) * 0.25
    bias = None if ta else seeded((n,), seed=23, dtype=dtype)
    av = _dev(a).t() if ta else _dev(a)
    bv = _dev(b).t() if tb else _dev(b)
    assert _ek().lib().tmb_gemm_workspace_bytes(1, m, n, k, _ops().code_of(dtype)) > 0
    got = _ops().gemm(av, bv, None if bias is None else _dev(bias))
    a64 = as64(a).T if ta else as64(a)
    b64 = as64(b).T if tb else as64(b)
    want = a64 @ b64 + (0 if bias is None else as64(bias))
    assert rel_frobenius(got, want) <= (1e-2 if dtype == torch.bfloat16 else 2e-3)
    ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    assert np.abs(as64(got) - want).max() <= ulp * np.abs(want).max() + 1e-3
    # one rounding: at most one storage ulp away from the kernel that does not split
    lib, ek = _ek().lib(), _ek()
    plain = torch.empty_like(got)
    ac, bc = av.contiguous() if ta else av, bv
    rc = lib.tmb_gemm(plain.data_ptr(), av.data_ptr(), bv.data_ptr(),
                      None if bias is None else _dev(bias).data_ptr(), 1, m, n, k,
                      a.shape[1], b.shape[1], n, 0, 0, m * n, int(ta), int(tb),
                      _ops().code_of(dtype), ek.EPI_NONE, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    del ac, bc
    assert np.abs(as64(got) - as64(plain)).max() <= 2 * ulp * np.abs(want).max() + 1e-3


def test_split_k_is_reproducible_and_needs_scratch_only_when_it_pays():
    lib = _ek().lib()
    code = _ops().code_of(torch.bfloat16)
    assert lib.tmb_gemm_workspace_bytes(1, 8192, 8192, 8192, code) == 0      # plenty of tiles
    assert lib.tmb_gemm_workspace_bytes(1, 1024, 768, 768, code) == 0        # short K
    assert lib.tmb_gemm_workspace_bytes(4, 1024, 768, 4096, code) == 0       # batched
    f32 = _ops().code_of(torch.float32)
    assert lib.tmb_gemm_workspace_bytes(1, 4096, 4096, 4096, f32) == 0       # fp32: plenty of tiles
    assert lib.tmb_gemm_workspace_bytes(1, 1024, 768, 4096, f32) == 8 * 1024 * 768 * 4
    a = _dev(seeded((512, 4096), seed=31, dtype=torch.bfloat16))
    b = _dev(seeded((4096, 384), seed=32, dtype=torch.bfloat16))
    first = _ops().gemm(a, b)
    for _ in range(3):
        assert torch.equal(first, _ops().gemm(a, b))


# ---- fp32 on the matrix cores --------------------------------------------------------------------
F32_LAYOUTS = [  # (m, n, k, trans_a, trans_b): aligned for the MFMA kernel, edges in every direction
    (128, 128, 16, False, False), (132, 260, 36, False, True), (132, 260, 36, True, False),
    (132, 260, 36, True, True), (4, 8, 4, False, False), (1, 772, 768, False, True),
    (300, 50257, 768, False, True), (257, 516, 1028, False, False), (257, 516, 1028, True, True),
    (128, 768, 3072, False, True), (128, 3072, 768, False, False), (16, 4096, 4096, False, True),
    (768, 768, 2048, True, False),
    (130, 131, 72, False, False), (130, 132, 70, False, True),   # unaligned: the SIMT kernel
]


@pytest.mark.parametrize("case", F32_LAYOUTS)
def test_fp32_mfma_all_layouts_match_float64(case):
    m, n, k, ta, tb = case
    a = seeded((k, m) if ta else (m, k), seed=41, dtype=torch.float32)
    b = seeded((n, k) if tb else (k, n), seed=42, dtype=torch.float32)
    bias = seeded((n,), seed=43, dtype=torch.float32)
    av = _dev(a).t() if ta else _dev(a)
    bv = _dev(b).t() if tb else _dev(b)
    got = _ops().gemm(av, bv, _dev(bias))
    a64 = as64(a).T if ta else as64(a)
    b64 = as64(b).T if tb else as64(b)
    want = a64 @ b64 + as64(bias)
    # fp32 products are exact in the accumulator's input; k additions round at 2^-24 each
    bound = k * 2.0 ** -24 * (np.abs(a64) @ np.abs(b64) + np.abs(as64(bias)))
    assert_close64(got, want, extra_abs=bound, what=f"fp32 gemm {case}")
    assert rel_frobenius(got, want) <= 2e-6


def test_fp32_mfma_batched_strided_and_gelu():
    a = _dev(seeded((6, 200, 96), seed=44, dtype=torch.float32))
    b = _dev(seeded((6, 96, 136), seed=45, dtype=torch.float32))
    got = _ops().gemm(a, b)
    want = as64(a) @ as64(b)
    assert rel_frobenius(got, want) <= 2e-6
    # rows of a wider buffer (lda > k) and a GELU epilogue against the separate kernel
    wide = _dev(seeded((200, 160), seed=46, dtype=torch.float32))
    a2 = wide[:, 32:128]
    w = _dev(seeded((136, 96), seed=47, dtype=torch.float32))
    bias = _dev(seeded((136,), seed=48, dtype=torch.float32))
    fused = _ops().gemm(a2, w.t(), bias, _ek().EPI_GELU_TANH, round_like_unfused=True)
    unfused = _ops().gelu(_ops().gemm(a2, w.t(), bias), "tanh")
    assert torch.equal(fused, unfused)
    assert torch.equal(fused, _ops().gemm(a2, w.t(), bias, _ek().EPI_GELU_TANH))   # float32: one mode
    want = as64(a2) @ as64(w).T + as64(bias)
    assert rel_frobenius(_ops().gemm(a2, w.t(), bias), want) <= 2e-6


def test_fp32_split_k_is_reproducible_and_close_to_the_unsplit_kernel():
    m, n, k = 128, 768, 3072
    lib, ek = _ek().lib(), _ek()
    assert lib.tmb_gemm_workspace_bytes(1, m, n, k, ek.F32) == 16 * m * n * 4
    a = _dev(seeded((m, k), seed=51, dtype=torch.float32))
    w = _dev(seeded((n, k), seed=52, dtype=torch.float32))
    bias = _dev(seeded((n,), seed=53, dtype=torch.float32))
    first = _ops().gemm(a, w.t(), bias)
    for _ in range(3):
        assert torch.equal(first, _ops().gemm(a, w.t(), bias))
    plain = torch.empty_like(first)
    rc = lib.tmb_gemm(plain.data_ptr(), a.data_ptr(), w.data_ptr(), bias.data_ptr(), 1, m, n, k,
                      k, k, n, 0, 0, m * n, 0, 1, ek.F32, ek.EPI_NONE,
                      torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    want = as64(a) @ as64(w).T + as64(bias)
    assert rel_frobenius(first, want) <= 2e-6 and rel_frobenius(plain, want) <= 2e-6


def test_fp32_mfma_output_larger_than_the_infinity_cache():
    """8192 x 8200 fp32 = 269 MB: the kernel's streaming-store path. Sampled rows against float64."""
    m, n, k = 8192, 8200, 64
    a = _dev(seeded((m, k), seed=61, dtype=torch.float32))
    w = _dev(seeded((n, k), seed=62, dtype=torch.float32))
    bias = _dev(seeded((n,), seed=63, dtype=torch.float32))
    got = _ops().gemm(a, w.t(), bias)
    rows = torch.tensor([0, 1, 127, 128, 4095, 4096, 8190, 8191], device="cuda")
    want = as64(a[rows]) @ as64(w).T + as64(bias)
    assert rel_frobenius(got[rows], want) <= 2e-6
    assert torch.isfinite(got).all()


# ---- K = 64 products on whole 128 x 128 tiles: the stream kernel -----------------------------------
# (batch, m, n): at least 512 tiles, so every persistent workgroup walks several of them; both
# layouts of B, a bias, a broadcast (stride 0) operand, and the shapes next to the kernel's limits
# that must take the general kernels instead.
STREAM64 = [(48, 1024, 1024), (8, 2048, 4096), (1, 4096, 8192), (96, 256, 768)]


@pytest.mark.parametrize("dtype", HALF)
@pytest.mark.parametrize("bmn", STREAM64)
@pytest.mark.parametrize("trans_b", [False, True])
def test_k64_stream_kernel_matches_float64(bmn, dtype, trans_b):
    batch, m, n = bmn
    g = torch.Generator(device="cuda").manual_seed(31)
    a = torch.randn(batch, m, 64, generator=g, device="cuda").to(dtype)
    b = torch.randn(batch, n, 64, generator=g, device="cuda").to(dtype)
    b = b.transpose(1, 2) if trans_b else b.transpose(1, 2).contiguous()
    if batch == 1:
        a, b = a[0], b[0]
    got = _ops().gemm(a, b)
    for sel in ((0,), (batch - 1,)) if batch > 1 else ((),):
        rows = torch.tensor([0, 31, 32, 127, 128, m // 2 + 5, m - 1], device="cuda")
        aa, bb, cc = (a[sel], b[sel], got[sel]) if batch > 1 else (a, b, got)
        aa, bb, cc = aa.reshape(m, 64), bb.reshape(64, n), cc.reshape(m, n)
        want = (aa[rows].double() @ bb.double()).cpu().numpy()
        bound = 64 * 2.0 ** -24 * (aa[rows].double().abs() @ bb.double().abs()).cpu().numpy()
        assert_close64(cc[rows], want, rtol=1e-6, atol=1e-6, extra_abs=bound, what=f"k64 {bmn} tb={trans_b}")
    # every tile was written: compare the whole product with the library kernel for K != 64
    # (same operands padded with zero columns take the general path)
    pad = torch.zeros(*a.shape[:-1], 8, device="cuda", dtype=dtype)
    a72 = torch.cat([a, pad], dim=-1)
    b72 = torch.cat([b, torch.zeros(*b.shape[:-2], 8, n, device="cuda", dtype=dtype)], dim=-2)
    assert torch.equal(got, _ops().gemm(a72, b72))


def test_k64_stream_kernel_bias_broadcast_and_neighbouring_shapes():
    g = torch.Generator(device="cuda").manual_seed(32)
    a = torch.randn(64, 512, 64, generator=g, device="cuda").bfloat16()
    w = torch.randn(64, 512, generator=g, device="cuda").bfloat16()       # one B for every batch entry
    got = _ops().gemm(a, w.unsqueeze(0).expand(64, 64, 512))
    want = (a.double() @ w.double())
    torch.testing.assert_close(got.double(), want, rtol=2.0 ** -7, atol=2.0 ** -6)
    # 2-D with a bias
    a2 = torch.randn(8192, 64, generator=g, device="cuda").bfloat16()
    b2 = torch.randn(64, 1024, generator=g, device="cuda").bfloat16()
    bias = torch.randn(1024, generator=g, device="cuda").bfloat16()
    got = _ops().gemm(a2, b2, bias)
    want = a2.double() @ b2.double() + bias.double()
    torch.testing.assert_close(got.double(), want, rtol=2.0 ** -7, atol=2.0 ** -6)
    # m not a multiple of 128, n not a multiple of 128, K = 32: the general kernels, same numbers
    for m, n, k in ((8200, 1024, 64), (8192, 1000, 64), (8192, 1024, 32)):
        x = torch.randn(m, k, generator=g, device="cuda").bfloat16()
        y = torch.randn(k, n, generator=g, device="cuda").bfloat16()
        torch.testing.assert_close(_ops().gemm(x, y).double(), x.double() @ y.double(),
                                   rtol=2.0 ** -7, atol=2.0 ** -6)
    # deterministic: three queued launches, identical bits
    outs = [_ops().gemm(a2, b2, bias) for _ in range(3)]
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])


# ---- operands the matrix-core kernels cannot read as they lie ------------------------------------
@pytest.mark.parametrize("case", [
    # (dtype, a shape, a transposed?, b shape, b transposed?)
    (torch.bfloat16, (700, 1001), False, (1001, 384), False),   # odd K: padded
    (torch.bfloat16, (1024, 1001), True, (1024, 256), False),   # weight-gradient form, odd M
    (torch.float16, (700, 1001), False, (384, 1001), True),     # odd K, K-major B
    (torch.bfloat16, (6, 512, 640), True, (6, 512, 64), False),  # transposed A, 64 columns
    (torch.float32, (600, 1001), False, (1001, 200), False),    # fp32, K not a multiple of 4
    (torch.float32, (1024, 1001), True, (1024, 128), False),    # fp32 weight-gradient form, odd M
])
def test_large_products_with_awkward_layouts_match_float64(case):
    """Above the re-layout threshold these run on the matrix-core kernels after one padded or
    transposed copy; the result is that of the product as given."""
    from torch_mojo_backend.eager_kernels import hip_ops
    dtype, ashape, ta, bshape, tb = case
    a = seeded(ashape, seed=41, dtype=dtype).cuda()
    b = seeded(bshape, seed=42, dtype=dtype).cuda()
    av = a.transpose(-1, -2) if ta else a
    bv = b.transpose(-1, -2) if tb else b
    m, k, n = av.shape[-2], av.shape[-1], bv.shape[-1]
    assert math.prod(av.shape[:-2]) * m * n * k >= hip_ops._RELAYOUT_MIN_WORK
    got = hip_ops.gemm(av, bv)
    want = as64(av) @ as64(bv)
    scale = np.abs(want).max()
    tol = {torch.float32: 2e-6, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype]
    assert np.abs(as64(got) - want).max() <= tol * scale
    ref = oracle.gemm(av.cpu(), bv.cpu())
    assert np.abs(as64(got) - as64(ref)).max() <= tol * scale


def test_pad_rows_kernel_matches_a_plain_copy():
    """Every alignment class of the source (odd pitches, odd offsets), 2- and 4-byte elements,
    3-D inputs with a constant row pitch; the padding is exact zeros."""
    from torch_mojo_backend.eager_kernels import hip_ops
    for dtype, shape, size in ((torch.bfloat16, (37, 1001), 1024), (torch.float16, (5, 9, 77), 80),
                               (torch.float32, (64, 50), 64), (torch.bfloat16, (3, 8), 8),
                               (torch.bfloat16, (129, 7), 64)):
        x = seeded(shape, seed=51, dtype=dtype).cuda()
        got = hip_ops._pad_last(x, size)
        assert got.is_contiguous() and got.shape[-1] == size
        assert torch.equal(got[..., : shape[-1]], x) and not got[..., shape[-1]:].any()
        # a view that starts at an odd element and has an odd pitch
        view = x[..., 1:]
        got = hip_ops._pad_last(view, size)
        assert torch.equal(got[..., : shape[-1] - 1], view) and not got[..., shape[-1] - 1:].any()
    # a transposed source is not row-major: PyTorch-ROCm's strided copy takes it
    x = seeded((40, 24), seed=52, dtype=torch.bfloat16).cuda().t()
    got = hip_ops._pad_last(x, 48)
    assert torch.equal(got[:, :40], x) and not got[:, 40:].any()
