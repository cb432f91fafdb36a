"""Pins for the oracle's scalar conversions: closed forms, exhaustive tables, stock torch."""
import numpy as np
import torch

from oracle import oracle as O
from oracle import torch_blocks as TB


def test_fp8_e4m3fn_closed_form_all_256():
    tab = O.fp8_table()
    for v in range(256):
        s, e, m = v >> 7, (v >> 3) & 15, v & 7
        if e == 15 and m == 7:
            assert np.isnan(tab[v])
            continue
        mag = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        assert tab[v] == np.float32(-mag if s else mag), v
    assert tab[0x7E] == 448.0 and tab[0xFE] == -448.0 and tab[0x01] == 2.0 ** -9
    assert not np.isinf(tab).any()


def test_fp8_table_matches_torch():
    tab = O.fp8_table()
    tt = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(tab), np.isnan(tt))
    ok = ~np.isnan(tab)
    assert np.array_equal(tab[ok].view(np.uint32), tt[ok].view(np.uint32))


def test_fp8_encode_matches_torch_and_roundtrips():
    L = O.lib()
    tab = O.fp8_table()
    for v in range(256):
        if np.isnan(tab[v]) or v == 0x80:
            continue
        assert L.orc_f32_to_fp8_e4m3fn(float(tab[v])) == v
    g = torch.Generator().manual_seed(0)
    for scale in (500.0, 1.0, 0.01):
        x = torch.randn(20000, generator=g) * scale
        x = x[x.abs() < 464.0]
        q = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        mine = np.array([L.orc_f32_to_fp8_e4m3fn(float(v)) for v in x.numpy()], np.uint8)
        assert np.array_equal(q, mine)


def test_bf16_rne_matches_torch():
    g = torch.Generator().manual_seed(1)
    a = torch.cat([torch.randn(200000, generator=g) * 3, torch.tensor([0.0, -0.0, 1.0, 1.00390625, 1.01171875,
                                                                        3.3895314e38, 1e-40, float("inf")])])
    assert np.array_equal(O.f32_to_bf16(a.numpy()), a.bfloat16().view(torch.int16).numpy().view(np.uint16))
    # ties to even: 1 + 2^-8 is halfway between 1 and 1 + 2^-7
    assert O.f32_to_bf16(np.float32([1 + 2.0 ** -8]))[0] == 0x3F80
    assert O.f32_to_bf16(np.float32([1 + 3 * 2.0 ** -8]))[0] == 0x3F82
    assert np.array_equal(O.bf16_to_f32(O.f32_to_bf16(a.numpy())), a.bfloat16().float().numpy(), equal_nan=True)


def test_dequant_closed_form_and_ragged():
    rng = np.random.default_rng(2)
    q = rng.integers(0, 256, size=(130, 200), dtype=np.uint8)
    q[(q & 0x7F) == 0x7F] = 0x3C
    s = (rng.random((2, 2)) * 0.02 + 1e-3).astype(np.float32)
    out = O.dequant_block(q, s)
    tab = O.fp8_table()
    exp = np.empty((130, 200), np.float32)
    for i in range(130):
        for j in range(200):
            exp[i, j] = np.float32(tab[q[i, j]]) * s[i // 128, j // 128]
    assert np.array_equal(out, O.f32_to_bf16(exp))
    tq = torch.from_numpy(q).view(torch.float8_e4m3fn)
    tt = TB.dequant(tq, torch.from_numpy(s))           # stock torch: repeat_interleave, trim, multiply, cast
    assert np.array_equal(out, tt.view(torch.int16).numpy().view(np.uint16))
    ones = np.ones((2, 2), np.float32)
    assert np.array_equal(O.bf16_to_f32(O.dequant_block(q, ones)), tab[q])   # every fp8 value is a bf16 value


def test_quantiser_matches_torch_and_error_bound():
    from moe_gen_amd.synthetic import quantize_fp8_block128
    g = torch.Generator().manual_seed(3)
    x = torch.randn(200, 300, generator=g) * 0.02
    q, s = O.quant_block(x.numpy())
    tq, ts = TB.quant(x)
    pq, ps = quantize_fp8_block128(x)
    assert np.array_equal(q, tq.view(torch.uint8).numpy()) and np.array_equal(s, ts.numpy())
    assert np.array_equal(q, pq.view(torch.uint8).numpy()) and np.array_equal(s, ps.numpy())
    deq = O.bf16_to_f32(O.dequant_block(q, s))
    xa = x.numpy()
    for bi in range(2):
        for bj in range(3):
            blk = (slice(bi * 128, (bi + 1) * 128), slice(bj * 128, (bj + 1) * 128))
            amax = max(np.abs(xa[blk]).max(), 1e-4)
            assert np.abs(deq[blk] - xa[blk]).max() <= amax * (2.0 ** -4 + 2.0 ** -8)
    z, zs = O.quant_block(np.zeros((5, 7), np.float32))
    assert (z == 0).all() and zs[0, 0] == np.float32(1e-4) / np.float32(448.0)


def test_canonical_exp_sigmoid_accuracy():
    xs = np.linspace(-104, 88.7, 1000001).astype(np.float32)
    ref = np.exp(xs.astype(np.float64))
    ulp = np.maximum(np.spacing(ref.astype(np.float32)).astype(np.float64), 1.4e-45)
    assert (np.abs(O.expf(xs).astype(np.float64) - ref) / ulp).max() <= 1.5
    assert O.expf(np.float32([0.0]))[0] == 1.0 and O.expf(np.float32([-200.0]))[0] == 0.0
    assert np.isinf(O.expf(np.float32([89.0]))[0])
    te = torch.exp(torch.from_numpy(xs)).numpy().astype(np.float64)
    assert (np.abs(O.expf(xs).astype(np.float64) - te) / ulp).max() <= 2.0
    zs = np.linspace(-30, 30, 200001).astype(np.float32)
    sref = 1.0 / (1.0 + np.exp(-zs.astype(np.float64)))
    sulp = np.spacing(sref.astype(np.float32)).astype(np.float64)
    assert (np.abs(O.sigmoidf(zs).astype(np.float64) - sref) / sulp).max() <= 2.5
    ts = torch.sigmoid(torch.from_numpy(zs)).numpy().astype(np.float64)
    assert (np.abs(O.sigmoidf(zs).astype(np.float64) - ts) / sulp).max() <= 4.0
