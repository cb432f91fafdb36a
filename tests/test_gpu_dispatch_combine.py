"""GPU parity of dispatch (histogram, offsets, stable permutation, gather) and combine."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from util import bf16_tensor, bits

pytestmark = pytest.mark.gpu


def rand_idx(n, k, E, seed, skew=False):
    rng = np.random.default_rng(seed)
    if skew:
        p = 1.0 / np.arange(1, E + 1) ** 1.2
        p /= p.sum()
    else:
        p = None
    return np.stack([rng.choice(E, size=k, replace=False, p=p) for _ in range(n)]).astype(np.int32)


@pytest.mark.parametrize("n,k,E", [(1, 1, 1), (7, 2, 8), (300, 6, 64), (2048, 8, 256), (5000, 6, 160),
                                   (4097, 2, 8), (33, 8, 256),
                                   (1536, 8, 256), (1537, 8, 256), (767, 16, 200)])   # either side of the one-workgroup form's 12288 entries
@pytest.mark.parametrize("skew", [False, True])
def test_dispatch_bit_exact(n, k, E, skew):
    from moe_gen_amd import ops
    print(f"dispatch n={n} k={k} E={E} skew={skew}", flush=True)
    idx = rand_idx(n, k, E, n + k + E, skew)
    h = 64
    x = torch.randn(n, h).to(torch.bfloat16)
    counts, offsets, perm, pos, xs, row_map = ops.dispatch(torch.from_numpy(idx).cuda(), E, x.cuda(), want_row_map=True)
    torch.cuda.synchronize()
    oc, oo, op, opos = O.dispatch(idx, E)
    assert np.array_equal(counts.cpu().numpy(), oc)
    assert np.array_equal(offsets.cpu().numpy(), oo)
    assert np.array_equal(perm.cpu().numpy(), op)
    assert np.array_equal(pos.cpu().numpy(), opos)
    assert np.array_equal(bits(xs), O.gather_rows(bits(x), op, k))
    assert np.array_equal(row_map.cpu().numpy(), op // k)


def test_dispatch_empty_and_unused_experts():
    from moe_gen_amd import ops
    idx = torch.zeros((0, 4), dtype=torch.int32, device="cuda")
    counts, offsets, perm, pos, _, _ = ops.dispatch(idx, 16)
    torch.cuda.synchronize()
    assert counts.sum().item() == 0 and offsets.sum().item() == 0 and perm.numel() == 0
    idx = torch.full((100, 1), 5, dtype=torch.int32, device="cuda")   # one expert takes everything
    counts, offsets, perm, pos, _, _ = ops.dispatch(idx, 16)
    assert counts.cpu().tolist() == [0] * 5 + [100] + [0] * 10
    assert perm.cpu().tolist() == list(range(100))


def test_dispatch_full_size_properties():
    """n*k = 524288 (the DeepSeek-V3 workload): integer identities instead of an oracle run."""
    from moe_gen_amd import ops
    n, k, E = 65536, 8, 256
    g = torch.Generator(device="cuda").manual_seed(3)
    idx = torch.rand((n, E), generator=g, device="cuda").topk(k, dim=1).indices.to(torch.int32)
    counts, offsets, perm, pos, _, row_map = ops.dispatch(idx, E, want_row_map=True)
    flat = idx.view(-1).long()
    assert torch.equal(counts.long(), torch.bincount(flat, minlength=E))
    assert torch.equal(offsets[1:].long(), counts.long().cumsum(0)) and offsets[0].item() == 0
    assert torch.equal(perm.long(), torch.argsort(flat, stable=True))
    assert torch.equal(pos[perm.long()].long(), torch.arange(n * k, device="cuda"))
    assert torch.equal(row_map, perm // k)


def test_dispatch_ignores_out_of_range_ids():
    """Ids outside [0, E) are not counted, own no sorted row and get pos -1, which the combine skips;
    the in-range entries are ranked as if the others were absent."""
    from moe_gen_amd import ops
    E, k = 16, 2
    idx = rand_idx(200, k, E, 5)
    bad = idx.copy()
    bad[3, 1], bad[77, 0], bad[199, 1] = 0x7fffffff, -1, E
    counts, offsets, perm, pos, _, _ = ops.dispatch(torch.from_numpy(bad).cuda(), E)
    torch.cuda.synchronize()
    flat = bad.reshape(-1)
    good = (flat >= 0) & (flat < E)
    assert np.array_equal(counts.cpu().numpy(), np.bincount(flat[good], minlength=E))
    n_good = int(good.sum())
    assert offsets.cpu().numpy()[-1] == n_good
    order = np.flatnonzero(good)[np.argsort(flat[good], kind="stable")]
    assert np.array_equal(perm.cpu().numpy()[:n_good], order)
    p = pos.cpu().numpy()
    assert np.array_equal(p[order], np.arange(n_good)) and (p[~good] == -1).all()
    # through the combine: a skipped slot adds nothing, i.e. the result equals the oracle's on a list in which
    # those slots point at a row of zeros with weight zero (x + 0 * 0 == x); the rows of y behind no slot hold NaN
    h = 256
    g = torch.Generator().manual_seed(3)
    ys = torch.full((flat.size, h), float("nan")).to(torch.bfloat16)
    ys[:n_good] = torch.randn(n_good, h, generator=g).to(torch.bfloat16)
    w = torch.rand(200, k, generator=g) * 2.5
    ys_ref = torch.cat([ys[:n_good], torch.zeros(1, h, dtype=torch.bfloat16)])
    pos_ref, w_ref, idx_ref = p.copy(), w.numpy().copy(), bad.copy()
    pos_ref[~good] = n_good
    w_ref.reshape(-1)[~good] = 0.0
    for mode in (0, 1, 2):
        out = ops.combine(ys.cuda(), pos, torch.from_numpy(bad).cuda(), w.cuda(), None, mode)
        torch.cuda.synchronize()
        ref = O.combine(bits(ys_ref), pos_ref, idx_ref, w_ref, None, mode)
        assert np.array_equal(bits(out), ref), mode


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("n,k,h,shared", [(1, 1, 8, False), (50, 2, 64, False), (257, 6, 2048, True),
                                          (100, 8, 7168, True), (33, 3, 5120, True), (9, 4, 8200, True),
                                          (5, 6, 16384, False)])   # 8200, 16384: more than one pass per block
def test_combine_bit_exact(mode, n, k, h, shared):
    from moe_gen_amd import ops
    print(f"combine mode={mode} n={n} k={k} h={h} shared={shared}", flush=True)
    E = 16
    idx = rand_idx(n, k, E, 11 * n + k)
    _, _, perm, pos = O.dispatch(idx, E)
    g = torch.Generator().manual_seed(n)
    ys = torch.randn(n * k, h, generator=g).to(torch.bfloat16)
    w = torch.rand(n, k, generator=g) * 2.5
    sh = torch.randn(n, h, generator=g).to(torch.bfloat16) if shared else None
    out = ops.combine(ys.cuda(), torch.from_numpy(pos).cuda(), torch.from_numpy(idx).cuda(), w.cuda(),
                      None if sh is None else sh.cuda(), mode)
    torch.cuda.synchronize()
    ref = O.combine(bits(ys), pos, idx, w.numpy(), None if sh is None else bits(sh), mode)
    assert np.array_equal(bits(out), ref), f"max abs diff {np.abs(O.bf16_to_f32(bits(out)) - O.bf16_to_f32(ref)).max()}"
