"""Host-side behaviour of the blocks that needs no GPU: parameter tree, errors, no CPU fallback."""
import pytest
import torch

import moe_gen_amd as M
from moe_gen_amd import deepseek_v2, synthetic


def tiny(family):
    w = {"v3": synthetic.WORKLOADS["deepseek_v3_w8a16"], "v2": synthetic.WORKLOADS["deepseek_v2_236b"],
         "mixtral": synthetic.WORKLOADS["mixtral_8x7b"]}[family]
    return w.scaled(n=16, h=128, I=128, E=8 if family != "v2" else 16, seq=4,
                    n_group=4 if family != "mixtral" else 1, topk_group=2 if family != "mixtral" else 1,
                    k=2)


def test_parameter_tree_matches_the_reference_names():
    """Keys the reference's initializers address (deepseekv3_initializer.py:1109-1152,
    Mixtral_Initializer.py:691-716)."""
    b3 = synthetic.build_block(tiny("v3"), device="cpu")
    keys = set(dict(b3.named_parameters()))
    for k in ("gate.weight", "gate.e_score_correction_bias", "experts.0.gate_proj.weight", "experts.7.down_proj.weight",
              "experts.3.up_proj.weight", "shared_experts.gate_proj.weight", "experts.0.gate_proj.weight_scale_inv"):
        assert k in keys, k
    assert b3.experts[0].gate_proj.weight.dtype == torch.float8_e4m3fn
    b2 = synthetic.build_block(tiny("v2"), device="cpu")
    assert {"gate.weight", "experts.15.up_proj.weight", "shared_experts.down_proj.weight"} <= set(dict(b2.named_parameters()))
    assert not hasattr(b2.gate, "e_score_correction_bias")
    assert b2.shared_experts.gate_proj.weight.shape == (2 * 128, 128)        # intermediate = S * I
    bm = synthetic.build_block(tiny("mixtral"), device="cpu")
    assert {"gate.weight", "experts.0.w1.weight", "experts.0.w2.weight", "experts.7.w3.weight"} <= set(dict(bm.named_parameters()))
    assert bm.experts[0].w1.weight.shape == (128, 128) and bm.gate.weight.shape == (8, 128)


def test_no_cpu_fallback():
    for fam in ("v3", "v2", "mixtral"):
        w = tiny(fam)
        blk = synthetic.build_block(w, device="cpu")
        with pytest.raises(RuntimeError, match="GPU"):
            blk(synthetic.hidden_states(w, "cpu"))
    with pytest.raises((RuntimeError, TypeError)):
        M.ops.router(torch.zeros(4, 16, dtype=torch.bfloat16), torch.zeros(8, 16, dtype=torch.bfloat16), None,
                     M.ops.RouterSpec(8, 2))


def test_unsupported_rules_raise_like_the_reference():
    cfg = M.DeepseekV3Config(hidden_size=64, n_routed_experts=8, n_group=2, topk_group=1, num_experts_per_tok=2,
                             moe_intermediate_size=64, scoring_func="softmax")
    blk = M.DeepseekV3MoE(cfg).eval()
    with pytest.raises(NotImplementedError, match="insupportable scoring function"):
        blk(torch.zeros(1, 2, 64, dtype=torch.bfloat16))
    cfg2 = M.DeepseekV2Config(hidden_size=64, n_routed_experts=8, num_experts_per_tok=2, moe_intermediate_size=64,
                              topk_method="gready")          # the reference config's own default (a typo upstream)
    gate = deepseek_v2.MoEGate(cfg2).eval()
    with pytest.raises(NotImplementedError, match="insupportable TopK function"):
        gate(torch.zeros(1, 2, 64, dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError):
        M.DeepseekV3MoE(M.DeepseekV3Config(hidden_size=64, n_routed_experts=8, ep_size=2, moe_intermediate_size=64))
    with pytest.raises(NotImplementedError):
        M.DeepseekV3MLP(M.DeepseekV3Config(hidden_size=64, intermediate_size=64, hidden_act="gelu"))


def test_workload_table_matches_the_benchmark_definition():
    W = synthetic.WORKLOADS
    v3 = W["deepseek_v3_w8a16"]
    assert (v3.n, v3.h, v3.E, v3.k, v3.I, v3.S, v3.n_group, v3.topk_group, v3.scale, v3.fp8) == \
        (65536, 7168, 256, 8, 2048, 1, 8, 4, 2.5, True)
    assert abs(v3.routed_flop - 46179.5e9) / 46179.5e9 < 1e-4 and abs(v3.shared_flop - 5772.4e9) / 5772.4e9 < 1e-4
    assert abs(v3.dispatch_bytes / 2 ** 20 - 14338) < 1 and abs(v3.combine_bytes / 2 ** 20 - 8962) < 1
    assert abs(v3.router_bytes / 2 ** 20 - 903.5) < 0.1
    v2 = W["deepseek_v2_236b"]
    assert (v2.n, v2.h, v2.E, v2.k, v2.I, v2.S, v2.method, v2.scale) == (32768, 5120, 160, 6, 1536, 2,
                                                                        "group_limited_greedy", 16.0)
    assert abs(W["mixtral_8x7b"].routed_flop - 11544.9e9) / 11544.9e9 < 1e-4
    assert W["mixtral_8x22b_decode"].n == 256 and W["deepseek_v2_lite"].zipf == 1.1


def test_zipf_bias_rides_on_feature_zero():
    w = synthetic.WORKLOADS["deepseek_v2_lite"].scaled(n=64, h=64)
    x = synthetic.hidden_states(w)
    g = synthetic.gate_weight(w)
    assert (x.reshape(-1, 64)[:, 0] == 1).all()
    b = g[:, 0].float()
    assert abs(b.mean().item()) < 0.02 and b.max() > 2.0 and b.min() < -0.5   # centred log-Zipf, skewed
    assert torch.equal(g, synthetic.gate_weight(w))                           # deterministic in the seed
