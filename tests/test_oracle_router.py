"""Pins for the oracle's router: exact cases, float64 ground truth, brute-force invariants,
stock-torch witnesses (oracle/torch_blocks.py uses torch's own softmax/sigmoid/topk)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle import torch_blocks as TB
from util import bf16_tensor, bits


def rand_inputs(n, h, E, seed, wscale=0.05):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    w = (torch.randn(E, h, generator=g) * wscale).to(torch.bfloat16)
    b = torch.randn(E, generator=g) * 0.01
    return x, w, b


def test_logits_exact_on_small_integers():
    """Integer-valued inputs: every partial sum is an exactly representable integer, so any
    dropped term, wrong index or transposed operand shows as an integer difference."""
    rng = np.random.default_rng(0)
    x = rng.integers(-8, 9, size=(7, 96)).astype(np.float32)
    w = rng.integers(-8, 9, size=(5, 96)).astype(np.float32)
    lg = O.logits(O.f32_to_bf16(x), O.f32_to_bf16(w))
    assert np.array_equal(lg, (x.astype(np.int64) @ w.astype(np.int64).T).astype(np.float32))


def test_logits_against_float64_bound():
    x, w, _ = rand_inputs(16, 7168, 32, 1, 0.02)
    lg = O.logits(bits(x), bits(w)).astype(np.float64)
    xd, wd = x.double().numpy(), w.double().numpy()
    exact = xd @ wd.T
    bound = 7168 * 2.0 ** -24 * (np.abs(xd) @ np.abs(wd).T)
    assert (np.abs(lg - exact) <= bound).all()
    assert np.abs(lg - exact).max() > 0        # it is an fp32 evaluation, not a float64 one


def test_softmax_scores_vs_torch():
    x, w, _ = rand_inputs(64, 256, 160, 2)
    spec = O.RouterSpec.deepseek_v2(160, 6)
    _, _, lg, sc = O.router(bits(x), bits(w), None, spec, want_scores=True)
    ts = torch.softmax(torch.from_numpy(lg), dim=-1, dtype=torch.float32).numpy()
    np.testing.assert_allclose(sc, ts, rtol=6e-7, atol=1e-12)
    np.testing.assert_allclose(sc.sum(axis=1), 1.0, atol=1e-6)


def test_sigmoid_scores_vs_torch():
    x, w, b = rand_inputs(64, 256, 64, 3, 0.2)
    spec = O.RouterSpec.deepseek_v3(64, 4, 4, 2)
    _, _, lg, sc = O.router(bits(x), bits(w), b.numpy(), spec, want_scores=True)
    np.testing.assert_allclose(sc, torch.sigmoid(torch.from_numpy(lg)).numpy(), rtol=5e-7)


def check_selection_invariants(lg, bias, spec):
    """From the definition, without re-running the selection: kept groups are the best groups,
    selected experts dominate unselected ones on the masked scores, ties resolve downwards."""
    idx, w, sc = O.router_from_logits(lg, bias, spec, want_scores=True)
    n, E = lg.shape
    k = spec.top_k
    c = sc + (bias if (spec.method == "noaux_tc" and bias is not None) else 0.0)
    c = c.astype(np.float32)
    for t in range(n):
        tmp = c[t].copy()
        if spec.method != "greedy":
            per = E // spec.n_group
            grp = c[t].reshape(spec.n_group, per)
            if spec.method == "noaux_tc":
                gs = np.sort(grp, axis=1)[:, -2:].astype(np.float32)
                gs = gs[:, 0] + gs[:, 1]
            else:
                gs = grp.max(axis=1)
            # brute force over all group subsets of size topk_group: best total, lowest indices on ties
            order = sorted(range(spec.n_group), key=lambda g: (-gs[g], g))
            kept = set(order[:spec.topk_group])
            mask = np.repeat([g in kept for g in range(spec.n_group)], per)
            tmp = np.where(mask, tmp, np.float32(0.0))
        sel = idx[t]
        assert len(set(sel.tolist())) == k
        uns = np.setdiff1d(np.arange(E), sel)
        if len(uns):
            assert tmp[sel].min() >= tmp[uns].max()
            for e in sel:                      # a selected expert never loses a tie to a lower index
                assert not ((tmp[uns] == tmp[e]) & (uns < e)).any()
        v = tmp[sel]
        assert all(v[j] > v[j + 1] or (v[j] == v[j + 1] and sel[j] < sel[j + 1]) for j in range(k - 1))
    return idx, w, sc


@pytest.mark.parametrize("spec", [
    O.RouterSpec.deepseek_v3(16, 4, 4, 2, True, 2.5),
    O.RouterSpec.deepseek_v3(256, 8, 8, 4, True, 2.5),
    O.RouterSpec.deepseek_v2(12, 3, "greedy"),
    O.RouterSpec.deepseek_v2(160, 6, "group_limited_greedy", 8, 3, False, 16.0),
    O.RouterSpec.mixtral(8, 2),
])
def test_selection_invariants_random_and_ties(spec):
    rng = np.random.default_rng(4)
    E = spec.n_experts
    lg = rng.normal(size=(40, E)).astype(np.float32)
    lg[10:20] = np.round(lg[10:20])            # many exact ties
    lg[20:24] = 0.0                            # everything ties
    lg[24:28, ::2] = lg[24:28, 1::2]           # pairwise ties
    bias = (rng.normal(size=E) * 0.01).astype(np.float32) if spec.method == "noaux_tc" else None
    idx, w, sc = check_selection_invariants(lg, bias, spec)
    if spec.method == "greedy":
        assert np.array_equal(idx[20], np.arange(spec.top_k))


def test_masked_experts_compete_with_zero():
    """Fewer than k positive candidates in the kept groups: masked experts (value 0.0) are picked,
    lowest index first, exactly like topk over masked_fill(~mask, 0.0) would allow."""
    spec = O.RouterSpec.deepseek_v3(8, 4, 4, 1, False, 1.0)      # 4 groups of 2, keep 1 group, k = 4
    lg = np.full((1, 8), -3.0, np.float32)
    lg[0, 4:6] = 3.0                                             # group 2 wins
    bias = np.zeros(8, np.float32)
    idx, w = O.router_from_logits(lg, bias, spec)
    assert idx[0].tolist() == [4, 5, 0, 1]
    np.testing.assert_allclose(w[0, 2:], 1 / (1 + np.exp(3.0)), rtol=1e-6)   # V3 gathers the true score
    spec2 = O.RouterSpec.deepseek_v2(8, 4, "group_limited_greedy", 4, 1, False, 1.0)
    idx2, w2 = O.router_from_logits(lg, None, spec2)
    assert idx2[0].tolist() == [4, 5, 0, 1] and (w2[0, 2:] == 0.0).all()     # V2 keeps the masked value


def test_weight_rules_v2_vs_v3():
    rng = np.random.default_rng(5)
    lg = rng.normal(size=(32, 16)).astype(np.float32)
    bias = np.zeros(16, np.float32)
    for norm in (True, False):
        for scale in (1.0, 16.0, 2.5):
            _, w3 = O.router_from_logits(lg, bias, O.RouterSpec.deepseek_v3(16, 4, 4, 2, norm, scale))
            _, w2 = O.router_from_logits(lg, None, O.RouterSpec.deepseek_v2(16, 4, "greedy", norm=norm, scale=scale))
            if norm:
                np.testing.assert_allclose(w3.sum(1), scale, rtol=1e-6)   # V3: normalise, then always scale
                np.testing.assert_allclose(w2.sum(1), 1.0, rtol=1e-6)     # V2: normalise INSTEAD of scaling
            else:
                _, w3u = O.router_from_logits(lg, bias, O.RouterSpec.deepseek_v3(16, 4, 4, 2, False, 1.0))
                _, w2u = O.router_from_logits(lg, None, O.RouterSpec.deepseek_v2(16, 4, "greedy", scale=1.0))
                np.testing.assert_allclose(w3, w3u * np.float32(scale), rtol=1e-7)
                np.testing.assert_allclose(w2, w2u * np.float32(scale), rtol=1e-7)
    # k == 1 never normalises
    _, w1 = O.router_from_logits(lg, None, O.RouterSpec.deepseek_v2(16, 1, "greedy", norm=True, scale=3.0))
    sc = torch.softmax(torch.from_numpy(lg), -1).numpy()
    np.testing.assert_allclose(w1[:, 0], sc.max(1) * 3.0, rtol=1e-6)


def near_tie_report(idx_o, idx_t, score_for_choice):
    """Tokens where two witnesses disagree must be near-ties of the selection score."""
    bad = np.nonzero((idx_o != idx_t).any(axis=1))[0]
    for t in bad:
        a, b = set(idx_o[t].tolist()), set(idx_t[t].tolist())
        d = list(a ^ b)
        s = score_for_choice[t]
        if d:
            assert np.ptp(s[d]) <= 1e-5 * max(1.0, np.abs(s[d]).max()), (t, s[d])
    return len(bad)


def test_v3_router_vs_stock_torch():
    n, h, E = 256, 512, 256
    x, w, b = rand_inputs(n, h, E, 6)
    spec = O.RouterSpec.deepseek_v3(E, 8, 8, 4, True, 2.5)
    idx, wt, lg, sc = O.router(bits(x), bits(w), b.numpy(), spec, want_scores=True)
    tidx, tw, tl = TB.gate_v3(x, w, b, 8, 8, 4, True, 2.5)
    np.testing.assert_allclose(lg, tl.numpy(), rtol=0, atol=2e-5)
    nbad = near_tie_report(idx, tidx.numpy(), sc + b.numpy())
    assert nbad <= n // 50
    same = (idx == tidx.numpy()).all(axis=1)
    np.testing.assert_allclose(wt[same], tw.numpy()[same], rtol=2e-5)


@pytest.mark.parametrize("method,G,Kg,norm,scale", [("greedy", 1, 1, False, 1.0),
                                                    ("group_limited_greedy", 8, 3, False, 16.0),
                                                    ("group_limited_greedy", 4, 2, True, 16.0)])
def test_v2_router_vs_stock_torch(method, G, Kg, norm, scale):
    n, h, E = 256, 512, 160 if G == 8 else 64
    x, w, _ = rand_inputs(n, h, E, 7)
    spec = O.RouterSpec.deepseek_v2(E, 6, method, G, Kg, norm, scale)
    idx, wt, lg, sc = O.router(bits(x), bits(w), None, spec, want_scores=True)
    tidx, tw, tl = TB.gate_v2(x, w, 6, method, G, Kg, norm, scale)
    nbad = near_tie_report(idx, tidx.numpy(), sc)
    assert nbad <= n // 50
    same = (idx == tidx.numpy()).all(axis=1)
    np.testing.assert_allclose(wt[same], tw.numpy()[same], rtol=3e-5)


def test_mixtral_router_vs_stock_torch():
    """bf16 gate: logits are bf16-rounded, so equal scores are common; with sorted top-k of torch
    the tie order is not specified, so compare where the top-3 scores are distinct."""
    n, h, E = 512, 512, 8
    x, w, _ = rand_inputs(n, h, E, 8)
    spec = O.RouterSpec.mixtral(E, 2)
    idx, wt, lg, sc = O.router(bits(x), bits(w), None, spec, want_scores=True)
    tidx, tw, tl = TB.gate_mixtral(x, w, 2)
    tl32 = tl.float().numpy()
    close = np.abs(lg - tl32) <= np.abs(tl32) * 2.0 ** -7      # at most one bf16 ulp apart (sum order)
    assert close.all()
    agree_l = (lg == tl32).all(axis=1)
    assert agree_l.mean() > 0.9
    top3 = np.sort(sc, axis=1)[:, -3:]
    distinct = (top3[:, 0] < top3[:, 1]) & (top3[:, 1] < top3[:, 2])
    m = agree_l & distinct
    assert m.sum() > n // 2
    assert np.array_equal(idx[m], tidx.numpy()[m])
    assert np.array_equal(O.f32_to_bf16(wt[m]), bits(tw)[m])    # weights are bf16 values
    assert (~distinct).sum() > 0                                 # ties really do occur with a bf16 gate


def test_golden_fixtures():
    """The committed vectors (tests/golden/*.npz, written by tests/golden/make_golden.py)."""
    import glob
    import os
    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "router_*.npz")))
    assert len(files) >= 4
    for f in files:
        z = np.load(f)
        spec = O.RouterSpec(**{k[5:]: z[k].item() for k in z.files if k.startswith("spec_")})
        bias = z["bias"] if "bias" in z.files else None
        idx, w, lg = O.router(z["x"], z["gate"], bias, spec)
        assert np.array_equal(idx, z["idx"]) and np.array_equal(w.view(np.uint32), z["w"].view(np.uint32)), f


def test_nan_scores_rank_above_every_number_as_in_torch_topk():
    """The reference hands NaN scores to torch.topk, which ranks NaN above every number.  The
    oracle's selections use that order (all NaNs equal, ties to the lower index), so the indices
    of a row with NaN scores are distinct and in range and the NaN reaches the weights."""
    rng = np.random.default_rng(11)
    E, k, n = 32, 4, 64
    lg = rng.normal(size=(n, E)).astype(np.float32)
    nan_at = [rng.choice(E, size=1 + t % 3, replace=False) for t in range(n)]
    for t, cols in enumerate(nan_at):
        lg[t, cols] = np.nan
    bias = (rng.normal(size=E) * 0.01).astype(np.float32)
    spec = O.RouterSpec.deepseek_v3(E, k, 1, 1, True, 2.5)          # one group: plain top-k of sigmoid + bias
    idx, w, sc = O.router_from_logits(lg, bias, spec, want_scores=True)
    c = torch.from_numpy(sc) + torch.from_numpy(bias)
    tidx = torch.topk(c, k, dim=-1).indices.numpy()
    for t in range(n):
        assert sorted(idx[t]) == sorted(tidx[t]), t                  # the library routine picks the same set
        m = len(nan_at[t])
        assert sorted(idx[t][:m]) == sorted(nan_at[t])               # NaNs first, in ascending index order
        assert list(idx[t][:m]) == sorted(idx[t][:m])
        assert np.isnan(w[t]).all()                                  # renormalised by a NaN sum
    # group-limited: a group that holds a NaN has a NaN group score and is kept first
    spec_g = O.RouterSpec.deepseek_v3(E, k, 4, 2, False, 1.0)
    idx, w = O.router_from_logits(lg, bias, spec_g)
    for t in range(n):
        assert len(set(idx[t])) == k and idx[t].min() >= 0 and idx[t].max() < E
        assert idx[t][0] == min(nan_at[t])
        assert np.isnan(w[t][0])
    # softmax: one NaN logit makes every score NaN; all equal -> the lowest indices in order
    idx, w = O.router_from_logits(lg, None, O.RouterSpec.deepseek_v2(E, k))
    assert (idx == np.arange(k)).all() and np.isnan(w).all()
    for G, Kg in ((4, 2), (8, 3)):
        idx, w = O.router_from_logits(lg, None, O.RouterSpec.deepseek_v2(E, k, "group_limited_greedy", G, Kg))
        assert (idx == np.arange(k)).all() and np.isnan(w).all()
