"""Pins for the oracle's RMSNorm and residual add (the steps either side of the MoE block)."""
import numpy as np
import torch

from oracle import oracle as O
from util import bf16_tensor, bits


def torch_rmsnorm(x, w, eps):
    """Stock-torch statement of DeepseekV3RMSNorm.forward (modeling_deepseek_v3.py:125-150)."""
    xf = x.to(torch.float32)
    var = xf.pow(2).mean(-1, keepdim=True)
    return w * (xf * torch.rsqrt(var + eps)).to(x.dtype)


def ulp_diff_bf16(a_bits, b_bits):
    """Distance in bf16 steps between two bit arrays of same-sign finite values."""
    return np.abs(a_bits.astype(np.int32) - b_bits.astype(np.int32))


def test_rmsnorm_against_stock_torch_and_float64():
    g = torch.Generator().manual_seed(0)
    for n, h, scale in ((5, 8, 1.0), (33, 2048, 1.0), (7, 7168, 30.0), (4, 4096, 1e-3)):
        x = (torch.randn(n, h, generator=g) * scale).to(torch.bfloat16)
        w = (1.0 + 0.1 * torch.randn(h, generator=g)).to(torch.bfloat16)
        got = O.rmsnorm(bits(x), bits(w), 1e-6)
        ref = bits(torch_rmsnorm(x, w, 1e-6))
        d = ulp_diff_bf16(got, ref)
        # torch's mean order and rsqrt differ from the canonical ones by a few fp32 ulps, which can
        # move a value across a bf16 rounding boundary, never further
        assert d.max() <= 1 and (d != 0).mean() < 2e-3, (n, h, d.max(), (d != 0).mean())
        # float64 ground truth of the two-rounding formula
        xf = x.double()
        rstd = 1.0 / torch.sqrt((xf * xf).mean(-1, keepdim=True) + 1e-6)
        y64 = (xf * rstd).to(torch.float32).to(torch.bfloat16)
        ref64 = bits((w.double() * y64.double()).to(torch.float32).to(torch.bfloat16))
        d = ulp_diff_bf16(got, ref64)
        assert d.max() <= 1 and (d != 0).mean() < 2e-3


def test_rmsnorm_closed_forms():
    h = 64
    one = bits(torch.ones(h, dtype=torch.bfloat16))
    # a constant row c normalises to c / sqrt(c^2 + eps): exactly sign(c) for eps = 0
    for c in (0.5, -3.0, 128.0):
        x = bits(torch.full((1, h), c, dtype=torch.bfloat16))
        out = O.bf16_to_f32(O.rmsnorm(x, one, 0.0))
        assert np.all(out == np.sign(c))
    # a one-hot row e_i * a normalises to sign(a) * sqrt(h) at position i (h = 64: exactly 8)
    x = torch.zeros(1, h); x[0, 5] = -7.0
    out = O.bf16_to_f32(O.rmsnorm(bits(x.to(torch.bfloat16)), one, 0.0))
    assert out[0, 5] == -8.0 and np.count_nonzero(out) == 1
    # an all-zero row stays zero (rstd = 1/sqrt(eps) is finite)
    assert not O.rmsnorm(bits(torch.zeros(2, h, dtype=torch.bfloat16)), one, 1e-6).any()
    # scaling the input by a power of two leaves the output unchanged when eps = 0
    g = torch.Generator().manual_seed(1)
    xr = torch.randn(3, 256, generator=g).to(torch.bfloat16)
    w = torch.randn(256, generator=g).to(torch.bfloat16)
    assert np.array_equal(O.rmsnorm(bits(xr), bits(w), 0.0), O.rmsnorm(bits(xr * 4), bits(w), 0.0))
    # the weight is applied after the rounding of the normalised value
    y = O.bf16_to_f32(O.rmsnorm(bits(xr), bits(torch.ones(256, dtype=torch.bfloat16)), 1e-6))
    assert np.array_equal(O.rmsnorm(bits(xr), bits(w), 1e-6), O.f32_to_bf16(O.bf16_to_f32(bits(w))[None, :] * y))


def test_add_residual_is_torch_bf16_add():
    g = torch.Generator().manual_seed(2)
    a = (torch.randn(50, 96, generator=g) * 3).to(torch.bfloat16)
    r = (torch.randn(50, 96, generator=g) * 50).to(torch.bfloat16)
    assert np.array_equal(O.add_residual(bits(a), bits(r)), bits(r + a))
    assert np.array_equal(O.add_residual(bits(a), bits(r)), O.add_residual(bits(r), bits(a)))


def test_golden_fixtures():
    """The committed vectors (tests/golden/rmsnorm_*.npz, written by tests/golden/make_golden.py)."""
    import glob
    import os
    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "rmsnorm_*.npz")))
    assert len(files) == 2
    for f in files:
        z = np.load(f)
        out = O.rmsnorm(z["x"], z["weight"], float(z["eps"]))
        assert np.array_equal(out, z["out"]), f
        assert np.array_equal(O.add_residual(out, z["residual"]), z["out_plus_residual"]), f
