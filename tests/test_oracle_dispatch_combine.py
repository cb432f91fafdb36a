"""Pins for the oracle's dispatch and combine: integer identities and library routines."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from util import bf16_tensor, bits


def rand_idx(n, k, E, seed):
    rng = np.random.default_rng(seed)
    return np.stack([rng.choice(E, size=k, replace=False) for _ in range(n)]).astype(np.int32)


@pytest.mark.parametrize("n,k,E", [(1, 1, 1), (100, 2, 8), (5000, 8, 256), (777, 6, 160)])
def test_dispatch_identities(n, k, E):
    idx = rand_idx(n, k, E, n)
    counts, offsets, perm, pos = O.dispatch(idx, E)
    flat = idx.reshape(-1)
    assert counts.sum() == n * k and np.array_equal(counts, np.bincount(flat, minlength=E))
    assert offsets[0] == 0 and np.array_equal(offsets[1:], np.cumsum(counts))
    assert np.array_equal(np.sort(perm), np.arange(n * k))                       # a bijection
    assert np.array_equal(perm, np.argsort(flat, kind="stable"))                 # numpy's stable sort
    assert np.array_equal(perm, torch.argsort(torch.from_numpy(flat).long(), stable=True).numpy())
    assert np.array_equal(pos[perm], np.arange(n * k))
    e_sorted = flat[perm]
    assert (np.diff(e_sorted) >= 0).all()
    for e in range(E):                                                            # ascending tokens per expert
        seg = perm[offsets[e]:offsets[e + 1]] // k
        assert (np.diff(seg) > 0).all()
    # the one-hot/scatter histogram of the reference (modeling_deepseek_v3.py:630-632)
    t = torch.from_numpy(idx).long()
    cn = t.new_zeros((n, E)); cn.scatter_(1, t, 1)
    assert np.array_equal(counts, cn.sum(0).numpy())


def test_dispatch_rejects_bad_index():
    with pytest.raises(ValueError):
        O.dispatch(np.array([[0, 9]], np.int32), 8)


def test_gather_rows():
    idx = rand_idx(50, 3, 10, 1)
    _, _, perm, _ = O.dispatch(idx, 10)
    x = torch.randn(50, 24).to(torch.bfloat16)
    xs = O.gather_rows(bits(x), perm, 3)
    assert np.array_equal(xs, bits(x[torch.from_numpy(perm).long() // 3]))


def setup_combine(n, k, h, seed):
    idx = rand_idx(n, k, 16, seed)
    _, _, perm, pos = O.dispatch(idx, 16)
    g = torch.Generator().manual_seed(seed)
    ys = torch.randn(n * k, h, generator=g).to(torch.bfloat16)
    w = (torch.rand(n, k, generator=g) * 2.5).float()
    sh = torch.randn(n, h, generator=g).to(torch.bfloat16)
    return idx, perm, pos, ys, w, sh


def test_combine_f32_closed_form_and_torch():
    n, k, h = 40, 4, 32
    idx, perm, pos, ys, w, sh = setup_combine(n, k, h, 3)
    out = O.combine(bits(ys), pos, idx, w.numpy(), None, O.COMBINE_F32)
    # the reference's own expression (modeling_deepseek_v3.py:702-710) with stock torch ops
    new_x = torch.empty_like(ys)
    new_x[torch.from_numpy(perm).long()] = ys
    ref = new_x.view(n, k, h).type(w.dtype).mul_(w.unsqueeze(-1)).sum(dim=1).type(new_x.dtype)
    d = np.abs(O.bf16_to_f32(out) - ref.float().numpy())
    assert (d <= np.abs(ref.float().numpy()) * 2.0 ** -7 + 1e-30).all()          # at most one bf16 ulp (sum order)
    assert (d == 0).mean() > 0.95
    exact = (ys.double()[torch.from_numpy(pos).long().view(n, k)] * w.double().unsqueeze(-1)).sum(1).numpy()
    assert np.abs(O.bf16_to_f32(out) - exact).max() <= np.abs(exact).max() * 2.0 ** -8
    out2 = O.combine(bits(ys), pos, idx, w.numpy(), bits(sh), O.COMBINE_F32)
    ref2 = ref + sh
    d2 = np.abs(O.bf16_to_f32(out2) - ref2.float().numpy())
    assert (d2 == 0).mean() > 0.9


def test_combine_uniform_weights_identical_rows():
    n, k, h = 9, 4, 16
    idx, perm, pos, ys, w, sh = setup_combine(n, k, h, 4)
    row = torch.randn(1, h).to(torch.bfloat16)
    ys = row.expand(n * k, h).contiguous()
    w = torch.full((n, k), 0.25)
    for mode in (O.COMBINE_F32, O.COMBINE_BF16_PROD, O.COMBINE_BF16_SEQ):
        out = O.combine(bits(ys), pos, idx, w.numpy(), None, mode)
        assert np.array_equal(out, bits(row.expand(n, h)))                        # 4 * (y/4) == y exactly


def test_combine_bf16_modes_vs_torch():
    n, k, h = 64, 2, 48
    idx, perm, pos, ys, w, sh = setup_combine(n, k, h, 5)
    new_x = torch.empty_like(ys)
    new_x[torch.from_numpy(perm).long()] = ys
    # V2 (modeling_deepseek_v2.py:744-757): weights cast to bf16, product and sum as bf16 tensors
    wb = w.to(torch.bfloat16)
    ref1 = new_x.view(n, k, h).mul(wb.unsqueeze(-1)).sum(dim=1)
    out1 = O.combine(bits(ys), pos, idx, w.numpy(), None, O.COMBINE_BF16_PROD)
    assert np.array_equal(out1, bits(ref1))
    # Mixtral: per expert in ascending id, index_add_ into a bf16 accumulator
    acc = torch.zeros(n, h, dtype=torch.bfloat16)
    for e in range(16):
        tok, slot = np.nonzero(idx == e)
        if len(tok):
            rows = torch.from_numpy(pos.reshape(n, k)[tok, slot]).long()
            cur = ys[rows] * wb[torch.from_numpy(tok), torch.from_numpy(slot), None]
            acc.index_add_(0, torch.from_numpy(tok), cur)
    out2 = O.combine(bits(ys), pos, idx, w.numpy(), None, O.COMBINE_BF16_SEQ)
    assert np.array_equal(out2, bits(acc))
