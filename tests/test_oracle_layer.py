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


def test_mixtral_layer_vs_installed_transformers():
    """A witness that is not this repository's: the MixtralSparseMoeBlock of the transformers package that happens to
    be installed (not the reference's pinned 4.42.0, which is absent: the router is the same published algorithm --
    bf16 gate Linear, softmax in fp32, top-k, renormalisation -- the experts are w1/w3/w2 as gate/up/down with SiLU,
    and tokens are added expert by expert in ascending id into a bf16 accumulator; newer releases keep the routing
    weights in fp32 where 4.42.0 rounds them to bf16 first, so outputs are compared to a bound, not bit for bit)."""
    tf = pytest.importorskip("transformers")
    mm = pytest.importorskip("transformers.models.mixtral.modeling_mixtral")
    if not hasattr(mm, "MixtralSparseMoeBlock"):
        pytest.skip("installed transformers has no MixtralSparseMoeBlock")
    n, h, I, E, k = 96, 256, 256, 8, 2
    x, gate, bias, experts, shared, lw = make("mixtral", n, h, I, E, k, False, 3)
    cfg = tf.MixtralConfig(hidden_size=h, intermediate_size=I, num_local_experts=E, num_experts_per_tok=k,
                           num_hidden_layers=1, num_attention_heads=4, num_key_value_heads=4, vocab_size=32)
    blk = mm.MixtralSparseMoeBlock(cfg).to(torch.bfloat16).eval()
    sd = blk.state_dict()
    names = set(sd)
    if {"gate.weight", "experts.gate_up_proj", "experts.down_proj"} <= names:      # fused expert tensors
        sd["gate.weight"].copy_(gate)
        sd["experts.gate_up_proj"].copy_(torch.stack([torch.cat([e[0], e[1]], 0) for e in experts]))
        sd["experts.down_proj"].copy_(torch.stack([e[2] for e in experts]))
    elif {"gate.weight", "experts.0.w1.weight"} <= names:                          # one module per expert
        sd["gate.weight"].copy_(gate)
        for e in range(E):
            sd[f"experts.{e}.w1.weight"].copy_(experts[e][0])
            sd[f"experts.{e}.w3.weight"].copy_(experts[e][1])
            sd[f"experts.{e}.w2.weight"].copy_(experts[e][2])
    else:
        pytest.skip(f"unknown parameter layout of the installed MixtralSparseMoeBlock: {sorted(names)[:6]}")
    with torch.no_grad():
        got = blk(x.clone())
    got = (got[0] if isinstance(got, tuple) else got).float().numpy().reshape(n, h)
    spec = O.RouterSpec.mixtral(E, k)
    out, aux = O.layer(bits(x).reshape(n, h), lw, spec, O.COMBINE_BF16_SEQ, rounding="ref")
    tidx = TB.gate_mixtral(x.view(n, h), gate, k)[0].numpy()
    same = (aux["idx"] == tidx).all(axis=1)               # rows whose bf16-logit ties torch orders the same way
    assert same.mean() > 0.8
    assert rel_max(O.bf16_to_f32(out)[same], got[same]) <= 1.2e-2
    # and the restatement this repository tests against elsewhere agrees with the package on every row
    ref, _ = TB.mixtral_block(x, gate, experts, k)
    assert rel_max(ref.float().numpy().reshape(n, h), got) <= 1.2e-2


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
