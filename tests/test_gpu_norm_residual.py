"""GPU parity of the steps either side of the block: RMSNorm kernel, residual add folded into the
combine, and the fused decoder-layer half against its unfused composition."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from test_gpu_dispatch_combine import rand_idx
from util import bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,h,scale", [(1, 8, 1.0), (3, 64, 1.0), (130, 2048, 1.0), (257, 7168, 20.0), (64, 4096, 1e-3),
                                       (5, 5120, 1.0), (9, 6144, 1.0), (7, 8192, 1.0), (6, 8200, 1.0),
                                       (3, 16384, 1.0)])   # 8200, 16384: rows too long to keep in registers
def test_rmsnorm_bit_exact(n, h, scale):
    from moe_gen_amd import ops
    print(f"rmsnorm n={n} h={h} scale={scale}", flush=True)
    g = torch.Generator().manual_seed(n + h)
    x = (torch.randn(n, h, generator=g) * scale).to(torch.bfloat16)
    x[0, : min(h, 16)] = 0
    w = (1.0 + 0.2 * torch.randn(h, generator=g)).to(torch.bfloat16)
    for eps in (1e-6, 1e-5):
        out = ops.rmsnorm(x.cuda(), w.cuda(), eps)
        torch.cuda.synchronize()
        assert np.array_equal(bits(out), O.rmsnorm(bits(x), bits(w), eps)), (n, h, eps)


def test_rmsnorm_edges_and_errors():
    from moe_gen_amd import ops
    w = torch.ones(64, dtype=torch.bfloat16, device="cuda")
    assert ops.rmsnorm(torch.zeros(0, 64, dtype=torch.bfloat16, device="cuda"), w).shape == (0, 64)
    z = ops.rmsnorm(torch.zeros(6, 64, dtype=torch.bfloat16, device="cuda"), w)
    assert not z.any()
    x = torch.randn(4, 64, device="cuda").to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="alias"):
        ops.rmsnorm(x, w, out=x)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        ops.rmsnorm(torch.zeros(2, 12, dtype=torch.bfloat16, device="cuda"), torch.ones(12, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(TypeError):
        ops.rmsnorm(x.float(), w)


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("n,k,h,shared,inplace", [(1, 1, 8, False, False), (50, 2, 64, False, True),
                                                  (257, 6, 2048, True, True), (100, 8, 7168, True, False)])
def test_combine_residual_bit_exact(mode, n, k, h, shared, inplace):
    from moe_gen_amd import ops
    print(f"combine_residual mode={mode} n={n} k={k} h={h} shared={shared} inplace={inplace}", flush=True)
    E = 16
    idx = rand_idx(n, k, E, 7 * n + k)
    _, _, perm, pos = O.dispatch(idx, E)
    g = torch.Generator().manual_seed(n + mode)
    ys = torch.randn(n * k, h, generator=g).to(torch.bfloat16)
    w = torch.rand(n, k, generator=g) * 2.5
    sh = torch.randn(n, h, generator=g).to(torch.bfloat16) if shared else None
    res = (torch.randn(n, h, generator=g) * 8).to(torch.bfloat16)
    res_d = res.cuda()
    out = ops.combine(ys.cuda(), torch.from_numpy(pos).cuda(), torch.from_numpy(idx).cuda(), w.cuda(),
                      None if sh is None else sh.cuda(), mode, out=res_d if inplace else None, residual=res_d)
    torch.cuda.synchronize()
    if inplace:
        assert out.data_ptr() == res_d.data_ptr()
    plain = O.combine(bits(ys), pos, idx, w.numpy(), None if sh is None else bits(sh), mode)
    assert np.array_equal(bits(out), O.add_residual(plain, bits(res)))


@pytest.mark.parametrize("name", ["deepseek_v3_w8a16", "deepseek_v2_lite", "mixtral_8x7b"])
def test_fused_decoder_half_equals_composition(name):
    """norm_moe_residual == residual + block(rmsnorm(residual)), bit for bit, and the norm it feeds
    the block is the oracle's."""
    from moe_gen_amd import norm_moe_residual, ops, synthetic
    w = synthetic.WORKLOADS[name].scaled(n=192, h=512, I=256, seq=64)
    blk = synthetic.build_block(w, device="cuda", gen_device="cpu")
    stream_in = (synthetic.hidden_states(w, "cpu") * 3).cuda()
    g = torch.Generator().manual_seed(5)
    ln = (1.0 + 0.1 * torch.randn(w.h, generator=g)).to(torch.bfloat16).cuda()
    xn = ops.rmsnorm(stream_in.view(-1, w.h), ln, 1e-6).view_as(stream_in)
    assert np.array_equal(bits(xn.view(-1, w.h)), O.rmsnorm(bits(stream_in.view(-1, w.h)), bits(ln), 1e-6))
    ref = blk(xn)
    fused = norm_moe_residual(blk, stream_in, ln, 1e-6)
    if isinstance(ref, tuple):
        assert torch.equal(fused[1], ref[1])
        ref, fused = ref[0], fused[0]
    torch.cuda.synchronize()
    assert fused.shape == stream_in.shape
    assert np.array_equal(bits(fused.view(-1, w.h)), O.add_residual(bits(ref.view(-1, w.h)), bits(stream_in.view(-1, w.h))))
    assert torch.equal(fused, stream_in + ref)
    assert getattr(blk, "_norm_residual", None) is None      # a later plain call is the plain block
    again = blk(xn)
    assert torch.equal(again[0] if isinstance(again, tuple) else again, ref)


def test_rmsnorm_golden_fixtures():
    """The committed vectors (tests/golden/rmsnorm_*.npz) through the C ABI: the norm kernel, and the
    residual add through the combine kernel with one slot of weight 1."""
    import glob
    import os
    from moe_gen_amd import ops
    from util import bf16_tensor
    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "rmsnorm_*.npz")))
    assert len(files) == 2
    for f in files:
        z = np.load(f)
        x, w, r = (bf16_tensor(z[k]).cuda() for k in ("x", "weight", "residual"))
        out = ops.rmsnorm(x, w, float(z["eps"]))
        assert np.array_equal(bits(out), z["out"]), f
        n = x.shape[0]
        ident = torch.arange(n, dtype=torch.int32, device="cuda")
        one = torch.ones(n, 1, device="cuda")
        summed = ops.combine(out, ident, None, one, None, ops.COMBINE_F32, residual=r)
        assert np.array_equal(bits(summed), z["out_plus_residual"]), f


def _fused_router_case(spec, has_bias, n, h, seed, eps=1e-6, scale=3.0):
    from moe_gen_amd import ops
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(n, h, generator=g) * scale).to(torch.bfloat16)
    ln = (1.0 + 0.1 * torch.randn(h, generator=g)).to(torch.bfloat16)
    wg = (torch.randn(spec.n_experts, h, generator=g) * 0.05).to(torch.bfloat16)
    bias = (torch.randn(spec.n_experts, generator=g) * 0.01) if has_bias else None
    s = ops.RouterSpec(**{f: getattr(spec, f) for f in ops.RouterSpec.__dataclass_fields__})
    idx, w, lg, xn = ops.router(x.cuda(), wg.cuda(), None if bias is None else bias.cuda(), s, True,
                                norm_weight=ln.cuda(), eps=eps)
    torch.cuda.synchronize()
    oxn = O.rmsnorm(bits(x), bits(ln), eps)
    assert np.array_equal(bits(xn), oxn), f"normalised rows differ (n={n} h={h} E={spec.n_experts})"
    oi, ow, ol = O.router(oxn, bits(wg), None if bias is None else bias.numpy(), spec)
    assert np.array_equal(lg.cpu().numpy().view(np.uint32), ol.view(np.uint32))
    assert np.array_equal(idx.cpu().numpy(), oi)
    assert np.array_equal(w.cpu().numpy().view(np.uint32), ow.view(np.uint32))


@pytest.mark.parametrize("n,h", [(300, 512), (64, 7168), (1, 64), (257, 1032), (130, 8200)])
def test_router_reading_through_the_norm_bit_exact(n, h):
    """moe_router_rmsnorm == oracle rmsnorm followed by the oracle router, bit for bit: normalised
    rows, logits, indices, weights; the three model families."""
    print(f"router through norm n={n} h={h}", flush=True)
    for spec, has_bias in ((O.RouterSpec.deepseek_v3(256, 8, 8, 4, True, 2.5), True),
                           (O.RouterSpec.deepseek_v2(160, 6, "group_limited_greedy", 8, 3, False, 16.0), False),
                           (O.RouterSpec.deepseek_v2(64, 6, "greedy", scale=1.0), False),
                           (O.RouterSpec.mixtral(8, 2), False)):
        _fused_router_case(spec, has_bias, n, h, 77 + n + h)


@pytest.mark.parametrize("E", [8, 16, 32, 48, 64, 96, 128, 144, 160, 176, 192, 208, 224, 256])
def test_router_through_norm_every_engine(E):
    """One case per logit engine and block layout (the token count picks them, as in the router's
    own bracket test): the norm pre-pass and the normalising stage store are part of each."""
    print(f"router through norm, engines, E={E}", flush=True)
    k = min(6, E)
    spec = O.RouterSpec.deepseek_v2(E, k, "greedy", scale=1.0)
    counts = [150, 4100 if E > 128 else 900, 8200 if E > 64 else 33000]
    if E <= 64:
        counts.append(65600)
    for n in counts:
        _fused_router_case(spec, False, n, 256, E + n, eps=1e-5, scale=0.5)


def test_router_through_norm_golden_and_errors():
    import glob
    import os
    from moe_gen_amd import ops
    from util import bf16_tensor
    spec = ops.RouterSpec(8, 2)
    for f in sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "rmsnorm_*.npz"))):
        z = np.load(f)
        x, w = (bf16_tensor(z[k]).cuda() for k in ("x", "weight"))
        gate = torch.zeros(8, x.shape[1], dtype=torch.bfloat16, device="cuda")
        xn = ops.router(x, gate, None, spec, norm_weight=w, eps=float(z["eps"]))[3]
        assert np.array_equal(bits(xn), z["out"]), f
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda")
    gate = torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        ops.router(x, gate, None, spec, norm_weight=torch.ones(32, dtype=torch.bfloat16, device="cuda"))
    out = ops.router(x[:0], gate, None, spec, norm_weight=torch.ones(64, dtype=torch.bfloat16, device="cuda"))
    assert out[3].shape == (0, 64)


def test_rmsnorm_sqrt_is_correctly_rounded():
    """A row whose var + eps has a square root that the hardware's approximate instruction gets
    1 ulp away from the correctly rounded value (sqrt(0x1.1531d8p-2)): rstd then differs by 1 ulp
    and two elements of the row round to other bf16 values.  The kernels use the correctly rounded
    square root, as the oracle does."""
    from moe_gen_amd import ops
    g = torch.Generator().manual_seed(158)
    x = (torch.randn(150, 256, generator=g) * 0.5).to(torch.bfloat16)
    ln = (1.0 + 0.1 * torch.randn(256, generator=g)).to(torch.bfloat16)
    want = O.rmsnorm(bits(x), bits(ln), 1e-5)
    assert np.array_equal(bits(ops.rmsnorm(x.cuda(), ln.cuda(), 1e-5)), want)
    gate = torch.zeros(8, 256, dtype=torch.bfloat16, device="cuda")
    assert np.array_equal(bits(ops.router(x.cuda(), gate, None, ops.RouterSpec(8, 2), norm_weight=ln.cuda(), eps=1e-5)[3]), want)
    # many rows, several eps: every rstd must match
    for seed, eps in ((1, 1e-5), (2, 1e-6), (3, 1e-3)):
        g = torch.Generator().manual_seed(seed)
        x = (torch.randn(8192, 64, generator=g) * (0.1 + seed)).to(torch.bfloat16)
        ln = torch.ones(64, dtype=torch.bfloat16)
        assert np.array_equal(bits(ops.rmsnorm(x.cuda(), ln.cuda(), eps)), O.rmsnorm(bits(x), bits(ln), eps)), (seed, eps)
