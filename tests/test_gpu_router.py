"""GPU parity of the fused router against the CPU oracle: indices AND weights bit-for-bit."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from util import bits

pytestmark = pytest.mark.gpu

FAMILIES = {
    "v3_256": (O.RouterSpec.deepseek_v3(256, 8, 8, 4, True, 2.5), True),
    "v3_nonorm": (O.RouterSpec.deepseek_v3(64, 4, 4, 2, False, 1.5), True),
    "v2_greedy_64": (O.RouterSpec.deepseek_v2(64, 6, "greedy", scale=1.0), False),
    "v2_group_160": (O.RouterSpec.deepseek_v2(160, 6, "group_limited_greedy", 8, 3, False, 16.0), False),
    "v2_group_norm": (O.RouterSpec.deepseek_v2(128, 6, "group_limited_greedy", 4, 2, True, 16.0), False),
    "mixtral_8": (O.RouterSpec.mixtral(8, 2), False),
    "greedy_24": (O.RouterSpec.deepseek_v2(24, 3, "greedy", scale=2.0), False),
}


def gpu_router(x, wg, bias, spec, want_logits=True):
    from moe_gen_amd import ops
    s = ops.RouterSpec(**{f: getattr(spec, f) for f in ops.RouterSpec.__dataclass_fields__})
    idx, w, lg = ops.router(x.cuda(), wg.cuda(), None if bias is None else bias.cuda(), s, want_logits)
    torch.cuda.synchronize()
    return idx.cpu().numpy(), w.cpu().numpy(), None if lg is None else lg.cpu().numpy()


@pytest.mark.parametrize("name", list(FAMILIES))
@pytest.mark.parametrize("n,h", [(300, 512), (64, 7168), (1, 64), (257, 1032)])
def test_router_bit_exact(name, n, h):
    spec, has_bias = FAMILIES[name]
    print(f"router case {name} n={n} h={h}", flush=True)
    g = torch.Generator().manual_seed(1234 + n + h)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    wg = (torch.randn(spec.n_experts, h, generator=g) * 0.05).to(torch.bfloat16)
    bias = (torch.randn(spec.n_experts, generator=g) * 0.01) if has_bias else None
    idx, w, lg = gpu_router(x, wg, bias, spec)
    oi, ow, ol = O.router(bits(x), bits(wg), None if bias is None else bias.numpy(), spec)
    assert np.array_equal(lg.view(np.uint32), ol.view(np.uint32)), \
        f"logits differ: max abs {np.abs(lg - ol).max()}"
    assert np.array_equal(idx, oi), f"{(idx != oi).any(axis=1).sum()} tokens with different indices"
    assert np.array_equal(w.view(np.uint32), ow.view(np.uint32)), f"weights differ: max abs {np.abs(w - ow).max()}"


@pytest.mark.parametrize("name", list(FAMILIES))
def test_router_forced_ties(name):
    """All-equal and pairwise-equal scores: ties go to the lower expert / group index."""
    spec, has_bias = FAMILIES[name]
    n, h, E = 96, 64, spec.n_experts
    g = torch.Generator().manual_seed(7)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    x[:32] = 0                                   # every logit 0 -> every score equal
    wg = (torch.randn(E, h, generator=g) * 0.05).to(torch.bfloat16)
    wg[1::2] = wg[0::2][: wg[1::2].shape[0]]     # experts 2i and 2i+1 identical -> pairwise ties
    bias = torch.zeros(E) if has_bias else None
    idx, w, _ = gpu_router(x, wg, bias, spec)
    oi, ow, _ = O.router(bits(x), bits(wg), None if bias is None else bias.numpy(), spec)
    assert np.array_equal(idx, oi)
    assert np.array_equal(w.view(np.uint32), ow.view(np.uint32))
    if spec.method == "greedy":
        assert np.array_equal(idx[0], np.arange(spec.top_k))


def test_router_large_shape_properties():
    """DeepSeek-V3 shape at 8192 tokens: invariants that need no oracle run."""
    spec, _ = FAMILIES["v3_256"]
    n, h = 8192, 7168
    g = torch.Generator().manual_seed(99)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    wg = (torch.randn(256, h, generator=g) * 0.02).to(torch.bfloat16)
    bias = torch.randn(256, generator=g) * 0.01
    idx, w, _ = gpu_router(x, wg, bias, spec, want_logits=False)
    assert idx.min() >= 0 and idx.max() < 256
    assert all(len(set(r)) == 8 for r in idx[:512])
    assert (np.unique(idx // 32, axis=1).shape[1] <= 8)
    groups = [len(set(r // 32)) for r in idx]
    assert max(groups) <= 4                                   # at most topk_group groups
    np.testing.assert_allclose(w.sum(axis=1), 2.5, rtol=1e-5)  # renormalised then scaled
    sub = slice(0, 128)
    oi, ow, _ = O.router(bits(x[sub]), bits(wg), bias.numpy(), spec)
    assert np.array_equal(idx[sub], oi) and np.array_equal(w[sub].view(np.uint32), ow.view(np.uint32))


def test_canonical_exp_sigmoid_on_device():
    """The device exp/sigmoid sequence equals the oracle's bit for bit (softmax of 1-hot rows
    exposes exp(l - max); sigmoid via the V3 path with zero bias)."""
    from moe_gen_amd import ops
    E, n = 64, 4096
    g = torch.Generator().manual_seed(5)
    # logits = x @ W^T with x = one-hot scaled rows: logit[t, e] = a_t * W[e, 0]
    vals = (torch.rand(n, generator=g) * 200 - 100).to(torch.bfloat16)
    x = torch.zeros(n, 8, dtype=torch.bfloat16); x[:, 0] = vals
    wg = torch.zeros(E, 8, dtype=torch.bfloat16); wg[:, 0] = torch.linspace(-1, 1, E).to(torch.bfloat16)
    for spec in (O.RouterSpec.deepseek_v2(E, 6), O.RouterSpec.deepseek_v3(E, 6, 4, 2, True, 1.0)):
        bias = torch.zeros(E) if spec.method == "noaux_tc" else None
        idx, w, lg = gpu_router(x, wg, bias, spec)
        oi, ow, ol = O.router(bits(x), bits(wg), None if bias is None else bias.numpy(), spec)
        assert np.array_equal(lg.view(np.uint32), ol.view(np.uint32))
        assert np.array_equal(idx, oi)
        assert np.array_equal(w.view(np.uint32), ow.view(np.uint32))


def test_router_and_dispatch_golden_fixtures():
    """The committed vectors (tests/golden/router_*.npz) through the C ABI."""
    import glob
    import os
    from moe_gen_amd import ops
    from util import bf16_tensor
    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "router_*.npz")))
    assert len(files) >= 4
    for f in files:
        z = np.load(f)
        spec = O.RouterSpec(**{k[5:]: z[k].item() for k in z.files if k.startswith("spec_")})
        bias = torch.from_numpy(z["bias"]) if "bias" in z.files else None
        idx, w, _ = gpu_router(bf16_tensor(z["x"]), bf16_tensor(z["gate"]), bias, spec)
        assert np.array_equal(idx, z["idx"]) and np.array_equal(w.view(np.uint32), z["w"].view(np.uint32)), f
        counts, offsets, perm, pos, _, _ = ops.dispatch(torch.from_numpy(idx).cuda(), spec.n_experts)
        assert np.array_equal(counts.cpu().numpy(), z["counts"]) and np.array_equal(perm.cpu().numpy(), z["perm"])
        assert np.array_equal(offsets.cpu().numpy(), z["offsets"]) and np.array_equal(pos.cpu().numpy(), z["pos"])


@pytest.mark.parametrize("E", [2, 4, 5, 8, 12, 16, 17, 32, 33, 64, 65, 96, 100, 128, 144, 160, 176, 192, 200, 224,
                               250, 256])
def test_every_expert_count_bracket(E):
    """One case per kernel instantiation (and an odd count inside it): greedy softmax routing and,
    where the count allows groups, sigmoid group-limited routing; logits, indices and weights
    bit-for-bit.  The token count picks the logit engine and its block layout inside a bracket:
    150 tokens (full tiles and a ragged one) the vector-ALU engine with a lane per (token, expert) pair up to
    16 experts, above that the 4x4 MFMA engine with 16 tokens per workgroup, above 64 experts the engine whose waves
    run without a common stage (4 tokens per workgroup); 4100 tokens (more than 128 experts) 16 per workgroup; 8200 tokens
    (more than 64 experts) the 32x32 MFMA engine (129 to 208 experts: with extra 4-expert groups per wave); up to 64 experts 33000 tokens the 4x4 engine with
    64 tokens per workgroup and 65600 the 32x32 engine (always 4x4 up to 16 experts)."""
    print(f"router bracket E={E}", flush=True)
    k = min(6, E)
    g = torch.Generator().manual_seed(E)
    specs = [(O.RouterSpec.deepseek_v2(E, k, "greedy", scale=1.0), False)]
    if E % 4 == 0 and E >= 16:
        specs.append((O.RouterSpec.deepseek_v3(E, k, 4, 2, True, 2.5), True))
    shapes = [(150, 136)]
    if E > 64:
        shapes.append((8200, 16))
        if E > 128:
            shapes.append((4100, 16))
    else:
        shapes.append((33000, 16))
        if E in (17, 32, 33, 64):
            shapes.append((65600, 16))
    for n, h in shapes:
        x = torch.randn(n, h, generator=g).to(torch.bfloat16)
        wg = (torch.randn(E, h, generator=g) * 0.1).to(torch.bfloat16)
        for spec, has_bias in specs:
            bias = (torch.randn(E, generator=g) * 0.01) if has_bias else None
            idx, w, lg = gpu_router(x, wg, bias, spec)
            oi, ow, ol = O.router(bits(x), bits(wg), None if bias is None else bias.numpy(), spec)
            assert np.array_equal(lg.view(np.uint32), ol.view(np.uint32)), (E, n, spec.method)
            assert np.array_equal(idx, oi), (E, n, spec.method)
            assert np.array_equal(w.view(np.uint32), ow.view(np.uint32)), (E, n, spec.method)


@pytest.mark.parametrize("E,n", [(96, 37), (256, 1024), (160, 1500), (256, 2048), (200, 1025)])
def test_barrier_free_engine_stage_counts(E, n):
    """More than 64 experts and few tokens: every wave streams its 64 gate rows through LDS buffers of its own, three
    of them up to 1024 tokens (the k loop unrolled by six stages of 64) and two up to 2048 tokens above 128 experts
    (unrolled by two).  Hidden sizes that leave 0 ... 5 whole stages after the unrolled loop, with and without a last
    stage of fewer than 64 k, and sizes below one stage; bit for bit against the oracle."""
    spec = O.RouterSpec.deepseek_v3(E, 6, 4, 2, True, 2.5) if E % 4 == 0 else O.RouterSpec.deepseek_v2(E, 6, "greedy")
    for h in (8, 56, 64, 72, 128, 384, 392, 448, 456, 576, 640, 704, 760):
        print(f"barrier-free engine E={E} n={n} h={h}", flush=True)
        g = torch.Generator().manual_seed(h + E)
        x = torch.randn(n, h, generator=g).to(torch.bfloat16)
        wg = (torch.randn(E, h, generator=g) * 0.1).to(torch.bfloat16)
        bias = (torch.randn(E, generator=g) * 0.01) if spec.method == "noaux_tc" else None
        idx, w, lg = gpu_router(x, wg, bias, spec)
        oi, ow, ol = O.router(bits(x), bits(wg), None if bias is None else bias.numpy(), spec)
        assert np.array_equal(lg.view(np.uint32), ol.view(np.uint32)), (E, n, h)
        assert np.array_equal(idx, oi), (E, n, h)
        assert np.array_equal(w.view(np.uint32), ow.view(np.uint32)), (E, n, h)


def test_router_random_shapes_at_switch_points():
    """Seeded random rules (expert count, top-k, family, groups) at token counts on both sides of
    every switch point of the logit engine's dispatch, bit-for-bit against the oracle."""
    import random
    rng = random.Random(7)
    edges = [1, 3, 4, 5, 7, 8, 9, 15, 16, 17, 63, 64, 65, 1023, 1024, 1025, 2047, 2048, 2049, 4095, 4096, 4097, 8191, 8192, 8193, 24576, 24577, 32768,
             32769, 65536, 65537]
    for it in range(56):
        E = rng.choice([1, 3, 7, 8, 9, 16, 20, 31, 32, 40, 50, 64, 72, 96, 120, 129, 160, 190, 208, 240, 256])
        k = rng.randint(1, min(E, 8))
        fam = rng.choice(["v2_greedy", "v2_group", "v3", "mixtral"])
        divs = [g for g in (2, 4, 8, 16) if E % g == 0 and E // g >= 2]
        if fam in ("v2_group", "v3") and not divs:
            fam = "v2_greedy"
        has_bias = False
        if fam == "v2_greedy":
            spec = O.RouterSpec.deepseek_v2(E, k, "greedy", scale=rng.choice([1.0, 16.0]), norm=rng.random() < 0.5)
        elif fam == "mixtral":
            spec = O.RouterSpec.mixtral(E, k)
        else:
            G = rng.choice(divs)
            Kg = rng.randint(1, G)
            k = min(k, Kg * (E // G))
            if fam == "v2_group":
                spec = O.RouterSpec.deepseek_v2(E, k, "group_limited_greedy", G, Kg, rng.random() < 0.5, 16.0)
            else:
                spec, has_bias = O.RouterSpec.deepseek_v3(E, k, G, Kg, rng.random() < 0.7, 2.5), True
        n = rng.choice(edges)
        h = 8 * rng.randint(1, 12)
        print(f"router random case {it}: E={E} k={k} {fam} n={n} h={h}", flush=True)
        g = torch.Generator().manual_seed(1000 + it)
        x = torch.randn(n, h, generator=g).to(torch.bfloat16)
        wg = (torch.randn(E, h, generator=g) * 0.1).to(torch.bfloat16)
        bias = (torch.randn(E, generator=g) * 0.01) if has_bias else None
        idx, w, lg = gpu_router(x, wg, bias, spec)
        oi, ow, ol = O.router(bits(x), bits(wg), None if bias is None else bias.numpy(), spec)
        assert np.array_equal(lg.view(np.uint32), ol.view(np.uint32)), (it, E, n, fam)
        assert np.array_equal(idx, oi), (it, E, n, fam)
        assert np.array_equal(w.view(np.uint32), ow.view(np.uint32)), (it, E, n, fam)


@pytest.mark.parametrize("name", ["v3_256", "mixtral_8", "v2_group_160", "v2_greedy_64"])
def test_router_nan_inputs_keep_indices_valid(name):
    """NaN in a token row or in a gate row: selections rank NaN above every number (torch.topk's
    order), so every lane group agrees, indices stay distinct and inside [0, E), and the NaN
    travels into the weights -- identical to the oracle; dispatch and combine then run on valid
    positions and the affected output rows are NaN."""
    from moe_gen_amd import ops
    spec, has_bias = FAMILIES[name]
    n, h, E, k = 200, 256, spec.n_experts, spec.top_k
    g = torch.Generator().manual_seed(21)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    wg = (torch.randn(E, h, generator=g) * 0.05).to(torch.bfloat16)
    bias = (torch.randn(E, generator=g) * 0.01) if has_bias else None
    x[3, 7] = float("nan"); x[150] = float("nan")          # whole rows of NaN logits
    wg[min(5, E - 1), 100] = float("nan")                    # one expert's logit is NaN for every token
    idx, w, _ = gpu_router(x, wg, bias, spec)
    oi, ow, _ = O.router(bits(x), bits(wg), None if bias is None else bias.numpy(), spec)
    assert idx.min() >= 0 and idx.max() < E and all(len(set(r)) == k for r in idx)
    assert np.array_equal(idx, oi)
    assert np.array_equal(np.isnan(w), np.isnan(ow))
    ok = ~np.isnan(ow)
    assert np.array_equal(w[ok].view(np.uint32), ow[ok].view(np.uint32))
    d = ops.dispatch(torch.from_numpy(idx).cuda(), E)
    y = torch.ones(n * k, 64, dtype=torch.bfloat16, device="cuda")
    out = ops.combine(y, d.pos, torch.from_numpy(idx).cuda(), torch.from_numpy(w).cuda(), None,
                      2 if name == "mixtral_8" else 0)
    torch.cuda.synchronize()
    assert np.array_equal(torch.isnan(out.float()).all(dim=1).cpu().numpy(), np.isnan(ow).any(axis=1))
