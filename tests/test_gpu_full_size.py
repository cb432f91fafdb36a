"""Full-size workloads (the shapes of the benchmark): properties that need no full oracle run,
plus an oracle check of a random subset of tokens."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from util import bits, oracle_spec, rel_max, weight_f32

pytestmark = pytest.mark.gpu

TOL = 2e-2


def subset_reference(blk, w, x2d, tokens, idx, wts):
    """fp32 oracle evaluation of the layer for the given token ids, using the routing the GPU chose
    (the routing itself is compared separately against the oracle's router)."""
    xf = O.bf16_to_f32(bits(x2d[tokens]))
    out = np.zeros((len(tokens), w.h), np.float32)
    cache = {}

    def mats(e):
        if e not in cache:
            cache[e] = tuple(weight_f32(p) for p in blk.experts[e].projections())
        return cache[e]

    for r, t in enumerate(tokens):
        for j in range(w.k):
            e = int(idx[t, j])
            out[r] += wts[t, j] * O.mlp_f32(xf[r:r + 1], *mats(e))[0]
    if w.S and w.family != "mixtral":
        out += O.mlp_f32(xf, *(weight_f32(p) for p in blk.shared_experts.projections()))
    return out


@pytest.mark.parametrize("name", ["deepseek_v3_w8a16", "deepseek_v2_236b", "mixtral_8x22b", "mixtral_8x7b",
                                  "deepseek_v2_lite", "mixtral_8x22b_decode"])
def test_full_size_layer(name):
    from moe_gen_amd import synthetic
    w = synthetic.WORKLOADS[name]
    print(f"full-size case {name}: n={w.n} h={w.h} E={w.E} k={w.k} I={w.I}", flush=True)
    blk = synthetic.build_block(w, device="cuda", gen_device="cuda")
    x = synthetic.hidden_states(w, "cuda")
    res = blk(x)
    out = (res[0] if isinstance(res, tuple) else res).view(w.n, w.h)
    torch.cuda.synchronize()
    x2d = x.view(w.n, w.h)
    idx, wts, counts = blk.last_topk_idx, blk.last_topk_weight, blk.last_counts
    # integer identities of routing and dispatch
    assert counts.sum().item() == w.n * w.k
    assert torch.equal(counts.long(), torch.bincount(idx.view(-1).long(), minlength=w.E))
    assert int(idx.min()) >= 0 and int(idx.max()) < w.E
    srt = torch.sort(idx, dim=1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all())                 # k distinct experts per token
    if w.family == "v3":
        torch.testing.assert_close(wts.sum(1), torch.full((w.n,), w.scale, device="cuda"), rtol=1e-5, atol=0)
        assert int(((idx // (w.E // w.n_group)).sort(1).values.diff(dim=1) != 0).sum(1).max()) + 1 <= w.topk_group
    assert torch.isfinite(out.float()).all()
    # token-permutation equivariance, bit for bit: every row is computed independently of its position
    g = torch.Generator(device="cuda").manual_seed(5)
    p = torch.randperm(w.n, generator=g, device="cuda")
    res2 = blk(x2d[p].contiguous().view(1, w.n, w.h))
    out2 = (res2[0] if isinstance(res2, tuple) else res2).view(w.n, w.h)
    assert torch.equal(out2, out[p])
    # routing of a random subset against the oracle (bit-exact), output against the fp32 oracle
    rng = np.random.default_rng(7)
    tokens = np.sort(rng.choice(w.n, size=24, replace=False))
    bias = blk.gate.e_score_correction_bias.data.cpu().numpy() if w.family == "v3" else None
    oi, ow, _ = O.router(bits(x2d[tokens]), bits(blk.gate.weight.data), bias, oracle_spec(w))
    idx_h, wts_h = idx.cpu().numpy(), wts.cpu().numpy()
    assert np.array_equal(idx_h[tokens], oi)
    assert np.array_equal(wts_h[tokens].view(np.uint32), ow.view(np.uint32))
    ref = subset_reference(blk, w, x2d, tokens, idx_h, wts_h)
    y = O.bf16_to_f32(bits(out[torch.from_numpy(tokens).cuda()]))
    err = rel_max(y, ref)
    print(f"  subset of 24 tokens: max-rel {err:.3e}", flush=True)
    assert err <= TOL
