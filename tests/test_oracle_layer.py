"""The oracle's whole layer against the stock-torch restatement of the reference blocks."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle import torch_blocks as TB
from util import bits, rel_max


def make(family, n, h, I, E, k, fp8, seed, S=0, **kw):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(1, n, h, generator=g).to(torch.bfloat16)
    gate = (torch.randn(E, h, generator=g) * 0.05).to(torch.bfloat16)
    bias = torch.randn(E, generator=g) * 0.01

    def mats(inter):
        out = []
        for shape in ((inter, h), (inter, h), (h, inter)):
            m = torch.randn(shape, generator=g) * 0.05
            out.append(TB.quant(m) if fp8 else m.to(torch.bfloat16))
        return tuple(out)

    experts = [mats(I) for _ in range(E)]
    shared = mats(S * I) if S else None

    def f32(m):
        if isinstance(m, tuple):
            return O.bf16_to_f32(O.dequant_block(bits(m[0]), m[1].numpy()))
        return O.bf16_to_f32(bits(m))

    lw = O.LayerWeights(bits(gate), bias.numpy() if family == "v3" else None,
                        [f32(e[0]) for e in experts], [f32(e[1]) for e in experts], [f32(e[2]) for e in experts],
                        tuple(f32(m) for m in shared) if shared else None)
    return x, gate, bias, experts, shared, lw


@pytest.mark.parametrize("fp8", [False, True])
def test_v3_layer_vs_torch_blocks(fp8):
    n, h, I, E, k = 96, 256, 128, 16, 4
    x, gate, bias, experts, shared, lw = make("v3", n, h, I, E, k, fp8, 1, S=1)
    spec = O.RouterSpec.deepseek_v3(E, k, 4, 2, True, 2.5)
    ref = TB.deepseek_block(x, gate, bias, experts, shared, "v3", k, "noaux_tc", 4, 2, True, 2.5, chunk=40)
    out, aux = O.layer(bits(x).reshape(n, h), lw, spec, O.COMBINE_F32, rounding="ref")
    o32, _ = O.layer(bits(x).reshape(n, h), lw, spec, O.COMBINE_F32, rounding="f32")
    r = ref.float().numpy().reshape(n, h)
    assert rel_max(O.bf16_to_f32(out), r) <= 1.2e-2       # same rounding points, different sum orders
    assert rel_max(r, o32) <= 2e-2                         # the torch restatement itself meets the bound


def test_v2_layer_vs_torch_blocks():
    n, h, I, E, k = 96, 256, 128, 16, 3
    x, gate, bias, experts, shared, lw = make("v2", n, h, I, E, k, False, 2, S=2)
    spec = O.RouterSpec.deepseek_v2(E, k, "group_limited_greedy", 4, 2, False, 4.0)
    ref = TB.deepseek_block(x, gate, None, experts, shared, "v2", k, "group_limited_greedy", 4, 2, False, 4.0)
    out, _ = O.layer(bits(x).reshape(n, h), lw, spec, O.COMBINE_BF16_PROD, rounding="ref")
    assert rel_max(O.bf16_to_f32(out), ref.float().numpy().reshape(n, h)) <= 1.2e-2


def test_mixtral_layer_vs_torch_blocks():
    n, h, I, E, k = 96, 256, 256, 8, 2
    x, gate, bias, experts, shared, lw = make("mixtral", n, h, I, E, k, False, 3)
    spec = O.RouterSpec.mixtral(E, k)
    ref, logits = TB.mixtral_block(x, gate, experts, k)
    out, aux = O.layer(bits(x).reshape(n, h), lw, spec, O.COMBINE_BF16_SEQ, rounding="ref")
    r = ref.float().numpy().reshape(n, h)
    tidx = TB.gate_mixtral(x.view(n, h), gate, k)[0].numpy()
    same = (aux["idx"] == tidx).all(axis=1)               # bf16-logit ties may be ordered differently by torch
    assert same.mean() > 0.8
    assert rel_max(O.bf16_to_f32(out)[same], r[same]) <= 1.2e-2


def test_dense_equivalence_k_equals_E():
    """k = E with identical experts and weights summing to 1: the layer is the dense MLP."""
    n, h, I, E = 32, 128, 64, 4
    x, gate, bias, experts, shared, lw = make("v2", n, h, I, E, E, False, 4)
    lw.wg, lw.wu, lw.wd = [lw.wg[0]] * E, [lw.wu[0]] * E, [lw.wd[0]] * E
    spec = O.RouterSpec.deepseek_v2(E, E, "greedy", norm=True)
    out, aux = O.layer(bits(x).reshape(n, h), lw, spec, rounding="f32")
    assert sorted(aux["counts"].tolist()) == [n] * E
    dense = O.mlp_f32(O.bf16_to_f32(bits(x)).reshape(n, h), lw.wg[0], lw.wu[0], lw.wd[0])
    assert rel_max(out, dense) <= 1e-5


def test_mlp_against_torch_linear():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(20, 64, generator=g).to(torch.bfloat16)
    wg, wu = [(torch.randn(48, 64, generator=g) * 0.1).to(torch.bfloat16) for _ in range(2)]
    wd = (torch.randn(64, 48, generator=g) * 0.1).to(torch.bfloat16)
    F = torch.nn.functional
    ref32 = F.linear(F.silu(F.linear(x.float(), wg.float())) * F.linear(x.float(), wu.float()), wd.float())
    f = lambda t: O.bf16_to_f32(bits(t))
    np.testing.assert_allclose(O.mlp_f32(f(x), f(wg), f(wu), f(wd)), ref32.numpy(), rtol=2e-4, atol=1e-6)
    refb = TB.swiglu(x, wg, wu, wd).float().numpy()
    assert rel_max(O.mlp_ref_rounding(f(x), f(wg), f(wu), f(wd)), refb) <= 1e-2
