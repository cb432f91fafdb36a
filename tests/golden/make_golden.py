"""Writes the small golden fixtures under tests/golden/ from the CPU oracle.

The reference repository holds no tests, vectors or fixtures for the MoE layer, and its Python
is not importable in this image (it needs transformers==4.42.0), so these vectors come from
oracle/moe_oracle.c; at generation time each is cross-checked against the stock-torch
restatement (oracle/torch_blocks.py) wherever the scores have no near-ties.

    python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from oracle import oracle as O  # noqa: E402
from oracle import torch_blocks as TB  # noqa: E402
from oracle import arena_format as AF  # noqa: E402
from util import bits  # noqa: E402


def router_case(name, spec, n, h, seed, has_bias):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    x[:8] = 0                                            # all scores tie
    w = (torch.randn(spec.n_experts, h, generator=g) * 0.05).to(torch.bfloat16)
    w[1] = w[0]                                          # experts 0 and 1 always tie
    b = (torch.randn(spec.n_experts, generator=g) * 0.01) if has_bias else None
    if b is not None:
        b[1] = b[0]
    idx, wt, lg = O.router(bits(x), bits(w), None if b is None else b.numpy(), spec)
    counts, offsets, perm, pos = O.dispatch(idx, spec.n_experts)
    # cross-check on the tie-free rows
    if spec.method == "noaux_tc":
        tidx = TB.gate_v3(x, w, b, spec.top_k, spec.n_group, spec.topk_group, spec.norm_topk_prob,
                          spec.routed_scaling_factor)[0].numpy()
    elif spec.logits_bf16:
        tidx = TB.gate_mixtral(x, w, spec.top_k)[0].numpy()
    else:
        tidx = TB.gate_v2(x, w, spec.top_k, spec.method, spec.n_group, spec.topk_group, spec.norm_topk_prob,
                          spec.routed_scaling_factor)[0].numpy()
    agree = (np.sort(idx[8:], 1) == np.sort(tidx[8:], 1)).all(1).mean()
    print(f"{name}: torch witness agrees on {agree:.0%} of the non-degenerate rows")
    assert agree > 0.7
    out = dict(x=bits(x), gate=bits(w), idx=idx, w=wt, counts=counts, offsets=offsets, perm=perm, pos=pos)
    if b is not None:
        out["bias"] = b.numpy()
    for f in ("n_experts", "top_k", "scoring", "method", "n_group", "topk_group", "norm_topk_prob", "scale_mode",
              "routed_scaling_factor", "norm_eps", "logits_bf16", "weights_bf16"):
        out["spec_" + f] = np.array(getattr(spec, f))
    np.savez_compressed(os.path.join(HERE, f"router_{name}.npz"), **out)


def main():
    router_case("v3", O.RouterSpec.deepseek_v3(64, 6, 8, 4, True, 2.5), 64, 64, 11, True)
    router_case("v2_greedy", O.RouterSpec.deepseek_v2(64, 6, "greedy", scale=1.0), 64, 64, 12, False)
    router_case("v2_group", O.RouterSpec.deepseek_v2(160, 6, "group_limited_greedy", 8, 3, False, 16.0), 64, 64, 13, False)
    router_case("mixtral", O.RouterSpec.mixtral(8, 2), 64, 64, 14, False)
    # fp8 decode table and one ragged dequantisation
    rng = np.random.default_rng(15)
    q = rng.integers(0, 256, size=(130, 200), dtype=np.uint8)
    q[(q & 0x7F) == 0x7F] = 0x3C
    s = (rng.random((2, 2)) * 0.02 + 1e-3).astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "fp8_dequant.npz"), table=O.fp8_table(), q=q, scale=s,
                        out=O.dequant_block(q, s))
    # RMSNorm (two row widths, one all-zero row, one large-magnitude row) and the residual add
    g = torch.Generator().manual_seed(16)
    for h in (64, 1544):
        x = torch.randn(9, h, generator=g).to(torch.bfloat16)
        x[0] = 0
        x[1] *= 300
        w = (1.0 + 0.2 * torch.randn(h, generator=g)).to(torch.bfloat16)
        r = torch.randn(9, h, generator=g).to(torch.bfloat16)
        out = O.rmsnorm(bits(x), bits(w), 1e-6)
        witness = bits(w * (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16))
        assert np.abs(out.astype(np.int32) - witness.astype(np.int32)).max() <= 1
        np.savez_compressed(os.path.join(HERE, f"rmsnorm_{h}.npz"), x=bits(x), weight=bits(w), eps=np.float32(1e-6),
                            out=out, residual=bits(r), out_plus_residual=O.add_residual(out, bits(r)))
    # weight-arena index on the wire: three modules, ragged tensor lists, a 0-dim and a 4-dim shape
    index = {"routed_expert_3_0": {"gate_proj.weight": (0, 29360128, (2048, 7168)),
                                   "gate_proj.weight_scale_inv": (29360128, 3584, (16, 56))},
             "shared_expert_3": {"down_proj.weight": (1 << 33, 12, (1, 2, 3, 2))},
             "lm_head": {"scalar": (40, 4, ())}}
    with open(os.path.join(HERE, "arena_index.bin"), "wb") as f:
        f.write(AF.serialize(index))
    with open(os.path.join(HERE, "arena_index.json"), "w") as f:
        json.dump({mk: {tk: [o, nb, list(sh)] for tk, (o, nb, sh) in inner.items()} for mk, inner in index.items()}, f,
                  indent=1)


if __name__ == "__main__":
    main()
