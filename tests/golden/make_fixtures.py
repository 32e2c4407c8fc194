"""Writes tests/golden/hot_ops_torch_cpu.npz: small seeded inputs with the outputs PyTorch CPU
eager gives for them.

PyTorch CPU eager is the yardstick the reference's own tests use for every hot op
(torch_mojo_backend/testing.py:186-229); the reference itself (Mojo/MAX) cannot run in this
environment and ships no stored vectors, so these fixtures come from PyTorch alone.
bfloat16 arrays are stored as their uint16 bit patterns (viewed as int16).

Run from the repository root:  python tests/golden/make_fixtures.py
"""

import os

import numpy as np
import torch


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy() if t.dtype == torch.bfloat16 else t.contiguous().numpy()


def main() -> None:
    g = torch.Generator().manual_seed(2026)
    out = {}
    x = torch.randn(33, 257, generator=g) * 4
    out["softmax_x"] = bits(x)
    out["softmax_y"] = bits(torch.softmax(x, -1))
    out["log_softmax_y"] = bits(torch.log_softmax(x, -1))

    ln_x = torch.randn(3, 65, generator=g).bfloat16()
    ln_w = (1 + 0.1 * torch.randn(65, generator=g)).bfloat16()
    ln_b = (0.1 * torch.randn(65, generator=g)).bfloat16()
    o, m, r = torch.native_layer_norm(ln_x, [65], ln_w, ln_b, 1e-5)
    out.update(ln_x=bits(ln_x), ln_w=bits(ln_w), ln_b=bits(ln_b), ln_out=bits(o),
               ln_mean=bits(m.float()), ln_rstd=bits(r.float()))

    ax = torch.randn(4, 50257, generator=g)
    for row, cols in ((1, (5, 40000)), (2, (0, 25000, 50256)), (3, (50255, 50256))):
        ax[row, list(cols)] = ax[row].max() + 1
    out["argmax_x"] = bits(ax)
    out["argmax_y"] = bits(torch.argmax(ax, dim=1))

    a = torch.randn(17, 24, generator=g).bfloat16()
    b = torch.randn(24, 40, generator=g).bfloat16()
    bias = torch.randn(40, generator=g).bfloat16()
    out.update(mm_a=bits(a), mm_b=bits(b), mm_bias=bits(bias), mm_out=bits(torch.addmm(bias, a, b)))

    sx = torch.randn(11, 1000, generator=g)
    out.update(sum_x=bits(sx), sum_rows=bits(sx.sum(1)), amax_rows=bits(sx.amax(1)))

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hot_ops_torch_cpu.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
