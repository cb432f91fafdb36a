"""GPU parity of the grouped SwiGLU GEMMs (bf16 and W8A16) and of the fp8 block dequantisation."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from util import bits, rel_max, rel_rms

pytestmark = pytest.mark.gpu

TOL = 2e-2     # max|y - y_ref| / max|y_ref| against the fp32 evaluation (bf16 inputs/weights)


def make_experts(E, h, I, fp8, seed):
    from moe_gen_amd.synthetic import quantize_fp8_block128
    g = torch.Generator().manual_seed(seed)
    mats = []
    for _ in range(E):
        one = []
        for shape in ((I, h), (I, h), (h, I)):
            m = torch.randn(shape, generator=g) * 0.05
            one.append(quantize_fp8_block128(m) if fp8 else m.to(torch.bfloat16))
        mats.append(one)
    return mats


def bits_t(t):
    return t.cpu().view(torch.int16)


def f32_of(m):
    if isinstance(m, tuple):
        return O.bf16_to_f32(O.dequant_block(bits(m[0]), m[1].numpy()))
    return O.bf16_to_f32(bits(m))


def run_case(E, h, I, counts, fp8, seed, use_row_map=False):
    from moe_gen_amd import ops
    counts = np.asarray(counts, np.int32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    n_rows = int(offsets[-1])
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(max(n_rows, 1), h, generator=g).to(torch.bfloat16)[:n_rows]
    mats = make_experts(E, h, I, fp8, seed + 1)
    dev = lambda m: tuple(t.cuda() for t in m) if isinstance(m, tuple) else m.cuda()
    dm = [[dev(m) for m in one] for one in mats]
    if fp8:
        ptrs = ops.expert_pointers([o[0][0] for o in dm], [o[1][0] for o in dm], [o[2][0] for o in dm],
                                   [o[0][1] for o in dm], [o[1][1] for o in dm], [o[2][1] for o in dm])
    else:
        ptrs = ops.expert_pointers([o[0] for o in dm], [o[1] for o in dm], [o[2] for o in dm])
    off_d = torch.from_numpy(offsets).cuda()
    if use_row_map:
        rm = torch.randperm(n_rows, generator=g).to(torch.int32)
        xin = torch.empty_like(x)
        xin[rm.long()] = x                       # row r of the sorted matrix lives at xin[rm[r]]
        y = ops.grouped_swiglu(xin.cuda(), rm.cuda(), ptrs, off_d, n_rows)
    else:
        y = ops.grouped_swiglu(x.cuda(), None, ptrs, off_d, n_rows)
    torch.cuda.synchronize()
    yf = O.bf16_to_f32(bits(y))
    xf = O.bf16_to_f32(bits(x))
    ref32 = np.zeros((n_rows, h), np.float32)
    refr = np.zeros((n_rows, h), np.float32)
    for e in range(E):
        a, b = offsets[e], offsets[e + 1]
        if b > a:
            wg, wu, wd = (f32_of(m) for m in mats[e])
            ref32[a:b] = O.mlp_f32(xf[a:b], wg, wu, wd)
            refr[a:b] = O.mlp_ref_rounding(xf[a:b], wg, wu, wd)
    return yf, ref32, refr


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("E,h,I,counts", [
    (1, 128, 128, [64]),
    (1, 256, 128, [300]),
    (4, 256, 384, [0, 1, 255, 257]),
    (8, 512, 256, [5, 0, 130, 64, 0, 0, 700, 31]),
    (3, 1024, 640, [1000, 3, 500]),
    (8, 256, 256, [3, 0, 40, 17, 0, 1, 64, 9]),        # every expert under a 64-row tile
    (6, 384, 128, [70, 2, 0, 33, 1, 5]),
    (2, 128, 128, [1, 0]),
    (4, 384, 256, [300, 500, 0, 260]),                 # 256-row tiles, ragged last N tile of the down projection
    (32, 256, 256, [3000] + [2] * 31),                 # one hot expert under a low mean: 24 tiles of 128 rows among 64-row tiles
])
def test_grouped_swiglu_vs_oracle(fp8, E, h, I, counts):
    print(f"grouped fp8={fp8} E={E} h={h} I={I} counts={counts}", flush=True)
    y, ref32, refr = run_case(E, h, I, counts, fp8, seed=17)
    assert np.isfinite(y).all()
    e32, er = rel_max(y, ref32), rel_max(y, refr)
    print(f"  max-rel vs fp32 {e32:.3e}  vs reference-rounding {er:.3e}  rms {rel_rms(y, ref32):.3e}", flush=True)
    assert e32 <= TOL
    assert er <= TOL


@pytest.mark.parametrize("E,h,I,counts", [
    (1, 192, 320, [300]),            # three 128-row tiles
    (2, 192, 320, [100, 30]),        # a 128-row tile and a 64-row tile
    (4, 320, 192, [5, 9, 0, 20]),    # 64-row tiles
    (1, 64, 64, [70]),               # a single k-stage
    (4, 384, 320, [300, 500, 0, 260]),   # gate/up: even stage count, ragged last N tile; down: 5 stages
])
def test_grouped_odd_stage_counts(E, h, I, counts):
    """bf16 sizes whose K is an odd multiple of 64: the k loop is unrolled by two and ends in a
    single-stage tail (fp8 sizes are multiples of 128 and never do)."""
    print(f"grouped odd stages E={E} h={h} I={I} counts={counts}", flush=True)
    y, ref32, _ = run_case(E, h, I, counts, False, seed=29)
    assert np.isfinite(y).all() and rel_max(y, ref32) <= TOL


@pytest.mark.parametrize("fp8", [False, True])
def test_tile_height_follows_the_expert(fp8):
    """One launch of the one-workgroup-per-tile kernel alone (mean rows per expert below 128) with experts on both
    sides of every tile-height boundary: a 64-row tile up to 64 rows, one 128-row tile up to 128, one 192-row
    tile up to 192, several 128-row tiles above (those share their weights through one XCD's L2).
    Against the oracle, and an expert's rows bit-for-bit against a launch that holds this expert alone."""
    from moe_gen_amd import ops
    E, h, I = 16, 512, 384
    counts = [3, 64, 65, 128, 129, 300, 0, 17, 257, 1, 192, 193, 1, 2, 0, 5]
    print(f"tile heights fp8={fp8} counts={counts}", flush=True)
    y, ref32, refr = run_case(E, h, I, counts, fp8, seed=61, use_row_map=True)
    assert np.isfinite(y).all() and rel_max(y, ref32) <= TOL and rel_max(y, refr) <= TOL
    # the same experts one at a time (run_case draws x and the weights from the seed alone)
    offsets = np.concatenate([[0], np.cumsum(counts)])
    mats = make_experts(E, h, I, fp8, 62)
    g = torch.Generator().manual_seed(61)
    x = torch.randn(int(offsets[-1]), h, generator=g).to(torch.bfloat16)
    dev = lambda m: tuple(t.cuda() for t in m) if isinstance(m, tuple) else m.cuda()
    for e in (1, 2):                                     # 64 and 65 rows: alone they are below a mean of 128 too
        one = [dev(m) for m in mats[e]]
        if fp8:
            ptrs = ops.expert_pointers([one[0][0]], [one[1][0]], [one[2][0]], [one[0][1]], [one[1][1]], [one[2][1]])
        else:
            ptrs = ops.expert_pointers([one[0]], [one[1]], [one[2]])
        a, b = int(offsets[e]), int(offsets[e + 1])
        ye = ops.grouped_swiglu(x[a:b].cuda(), None, ptrs, torch.tensor([0, b - a], dtype=torch.int32, device="cuda"), b - a)
        torch.cuda.synchronize()
        assert np.array_equal(O.bf16_to_f32(bits(ye)), y[a:b]), f"expert {e} differs from its launch alone"


@pytest.mark.parametrize("fp8", [False, True])
def test_experts_split_between_the_two_kernels(fp8):
    """From a mean of 128 rows per expert a call launches both kernels and every expert goes by its own count.  bf16
    weights: up to 192 rows one tile of the one-workgroup-per-tile kernel, more the persistent kernel's 256-row tiles.
    fp8 weights: the persistent kernel's tile space holds an expert's full 256-row tiles, and what they leave over goes
    to the other kernel if it is at most 192 rows (300 = 256 + 44, 640 = 512 + 128, 700 = 512 + 188, 512 leaves nothing,
    2000 = 1792 + 208 stays whole).  (At this size the tile space is a short last round, which the other kernel runs as half tiles.)
    Against the oracle, and every expert's rows bit-for-bit against a call that holds this expert alone, whichever
    kernel and tile its rows fall to there.  (A lone call below a mean of 128 is served by the one-workgroup-per-tile
    kernel alone, which then walks k from other stages than a call of both kernels, and is left out.)"""
    from moe_gen_amd import ops
    E, h, I = 13, 256, 384
    counts = [700, 3, 192, 193, 64, 0, 129, 2000, 128, 300, 512, 640, 1600]
    print(f"two kernels fp8={fp8} counts={counts}", flush=True)
    y, ref32, refr = run_case(E, h, I, counts, fp8, seed=71, use_row_map=True)
    assert np.isfinite(y).all() and rel_max(y, ref32) <= TOL and rel_max(y, refr) <= TOL
    offsets = np.concatenate([[0], np.cumsum(counts)])
    mats = make_experts(E, h, I, fp8, 72)
    g = torch.Generator().manual_seed(71)
    x = torch.randn(int(offsets[-1]), h, generator=g).to(torch.bfloat16)
    dev = lambda m: tuple(t.cuda() for t in m) if isinstance(m, tuple) else m.cuda()
    for e in range(E):
        a, b = int(offsets[e]), int(offsets[e + 1])
        if b - a < 128:
            continue
        one = [dev(m) for m in mats[e]]
        if fp8:
            ptrs = ops.expert_pointers([one[0][0]], [one[1][0]], [one[2][0]], [one[0][1]], [one[1][1]], [one[2][1]])
        else:
            ptrs = ops.expert_pointers([one[0]], [one[1]], [one[2]])
        ye = ops.grouped_swiglu(x[a:b].cuda(), None, ptrs, torch.tensor([0, b - a], dtype=torch.int32, device="cuda"), b - a)
        torch.cuda.synchronize()
        assert np.array_equal(O.bf16_to_f32(bits(ye)), y[a:b]), f"expert {e} ({b - a} rows) differs from its call alone"


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("I,counts", [(1280, [700, 520, 300, 1300, 90]),      # gate/up: less than half a round
                                      (2048, [700, 520, 300, 1300, 90]),      # gate/up: 192 tiles next to 48 of the other kernel
                                      (2560, [700, 520, 300, 1300, 90]),      # gate/up: a round and a few tiles
                                      (1664, [2100, 2300, 2500, 1500, 10])])  # gate/up: 442 tiles, a round + 186, next to 13
def test_rounds_of_the_persistent_kernel_and_its_last_tiles(fp8, I, counts):
    """The persistent kernel (one workgroup per CU) takes whole rounds of 256 tiles; its last, partial round goes to
    the other kernel as 128-row halves when that shortens the two launches: alone, a round of at most 128 tiles;
    next to the other kernel's own tiles also a longer one (192 + 48 tiles: one launch of 432 half and whole tiles
    instead of two launches; 186 of 442 likewise).  Tile counts in the comments are for bf16 weights (with fp8
    weights only an expert's full tiles and ragged tiles above 128 rows count).  The down projections of these cases
    have a few dozen tiles, all of them half tiles.  Against the oracle."""
    from moe_gen_amd import ops
    E, h = len(counts), 256
    print(f"rounds fp8={fp8} I={I} counts={counts}", flush=True)
    y, ref32, refr = run_case(E, h, I, counts, fp8, seed=91, use_row_map=True)
    assert np.isfinite(y).all() and rel_max(y, ref32) <= TOL and rel_max(y, refr) <= TOL


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("counts", [[300, 640, 129, 70], [2100, 1700], [40, 3, 77]])
def test_a_row_does_not_depend_on_its_place_in_its_expert(fp8, counts):
    """The same rows in another order within every expert give the same output rows, bit for bit, whichever kernel
    and tile a row falls to (with fp8 weights the rows past an expert's last full 256-row tile are computed by the
    other kernel: 300 = 256 + 44)."""
    from moe_gen_amd import ops
    E, h, I = len(counts), 256, 384
    print(f"row order fp8={fp8} counts={counts}", flush=True)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    n = int(offsets[-1])
    g = torch.Generator().manual_seed(83)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    perm = torch.cat([int(offsets[e]) + torch.randperm(counts[e], generator=g) for e in range(E)])
    mats = make_experts(E, h, I, fp8, 84)
    dev = lambda m: tuple(t.cuda() for t in m) if isinstance(m, tuple) else m.cuda()
    dm = [[dev(m) for m in one] for one in mats]
    if fp8:
        ptrs = ops.expert_pointers([o[0][0] for o in dm], [o[1][0] for o in dm], [o[2][0] for o in dm],
                                   [o[0][1] for o in dm], [o[1][1] for o in dm], [o[2][1] for o in dm])
    else:
        ptrs = ops.expert_pointers([o[0] for o in dm], [o[1] for o in dm], [o[2] for o in dm])
    off_d = torch.from_numpy(offsets).cuda()
    y1 = ops.grouped_swiglu(x.cuda(), None, ptrs, off_d, n)
    y2 = ops.grouped_swiglu(x[perm].cuda(), None, ptrs, off_d, n)
    y3 = ops.grouped_swiglu(x.cuda(), perm.to(torch.int32).cuda(), ptrs, off_d, n)       # the same through a row map
    torch.cuda.synchronize()
    assert torch.equal(y2, y1[perm.cuda()])
    assert torch.equal(y3, y2)


@pytest.mark.parametrize("h,I", [(512, 384), (2048, 1024)])
def test_fp8_weight_streamer_rows_do_not_depend_on_the_tile(h, I):
    """fp8 experts of up to 64 rows, in a call below a mean of 128 rows per expert, go through the weight streamer
    (weights by DMA as fp8, one 16/32/48/64-row body per expert).  Eight experts that share one set of weights and
    hold 5 ... 64 rows, each starting with the same five rows: those rows come out bit-identical from every body,
    against the oracle within the layer bound, and the call gives the same bits every time it runs (the buffers of
    a tile are refilled while other waves still multiply; a missing wait shows as run-to-run differences)."""
    from moe_gen_amd import ops
    counts = [5, 16, 17, 32, 33, 48, 49, 64]
    E = len(counts)
    print(f"fp8 streamer h={h} I={I} counts={counts}", flush=True)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    n = int(offsets[-1])
    g = torch.Generator().manual_seed(97)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    for e in range(1, E):
        x[offsets[e]:offsets[e] + 5] = x[:5]
    one = make_experts(1, h, I, True, 98)[0]
    dm = [tuple(t.cuda() for t in m) for m in one]
    ptrs = ops.expert_pointers([dm[0][0]] * E, [dm[1][0]] * E, [dm[2][0]] * E, [dm[0][1]] * E, [dm[1][1]] * E, [dm[2][1]] * E)
    off_d = torch.from_numpy(offsets).cuda()
    xd = x.cuda()
    ys = [ops.grouped_swiglu(xd, None, ptrs, off_d, n).clone() for _ in range(8)]
    torch.cuda.synchronize()
    for rep in range(1, 8):
        assert torch.equal(ys[rep], ys[0]), f"call {rep} differs from call 0"
    for e in range(1, E):
        assert torch.equal(ys[0][offsets[e]:offsets[e] + 5], ys[0][:5]), f"expert {e} ({counts[e]} rows)"
    wg, wu, wd = (f32_of(m) for m in one)
    ref = O.mlp_f32(O.bf16_to_f32(bits(x)), wg, wu, wd)
    assert rel_max(O.bf16_to_f32(bits(ys[0])), ref) <= TOL


@pytest.mark.parametrize("counts", [
    [5, 16, 17, 32, 33, 64, 65, 80, 81, 96, 112, 128, 129, 144, 160, 176, 192] + [5] * 12,     # mean 59: one kernel
    [192, 181, 170, 160, 150, 140, 130, 129, 257, 300, 384, 600, 5]])                          # mean 215: both kernels
def test_bf16_weight_streamer_rows_do_not_depend_on_the_tile(counts):
    """bf16 experts of up to 192 rows (and the halves of one of 257 ... 384) go through the bf16 weight streamer: one
    body per number of 16-row groups, two wave layouts (up to 64 rows, above), weights and token rows by DMA.
    Experts that share one set of weights and start with the same five rows: those rows come out bit-identical from
    every body -- in the second list also from the persistent kernel (600 rows) and the halves of a pair --, against
    the oracle within the layer bound, and the call gives the same bits every time it runs (a tile's buffers are
    refilled while other waves still multiply; a missing wait shows as run-to-run differences)."""
    from moe_gen_amd import ops
    E, h, I = len(counts), 448, 640            # 7 / 10 stages of 64 k: 1 / 4 stages after the loop unrolled by six
    print(f"bf16 streamer counts={counts}", flush=True)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    n = int(offsets[-1])
    g = torch.Generator().manual_seed(197)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    for e in range(1, E):
        x[offsets[e]:offsets[e] + 5] = x[:5]
    one = make_experts(1, h, I, False, 198)[0]
    dm = [m.cuda() for m in one]
    ptrs = ops.expert_pointers([dm[0]] * E, [dm[1]] * E, [dm[2]] * E)
    off_d = torch.from_numpy(offsets).cuda()
    xd = x.cuda()
    ys = [ops.grouped_swiglu(xd, None, ptrs, off_d, n).clone() for _ in range(8)]
    torch.cuda.synchronize()
    for rep in range(1, 8):
        assert torch.equal(ys[rep], ys[0]), f"call {rep} differs from call 0"
    for e in range(1, E):
        assert torch.equal(ys[0][offsets[e]:offsets[e] + 5], ys[0][:5]), f"expert {e} ({counts[e]} rows)"
    wg, wu, wd = (f32_of(m) for m in one)
    ref = O.mlp_f32(O.bf16_to_f32(bits(x)), wg, wu, wd)
    assert rel_max(O.bf16_to_f32(bits(ys[0])), ref) <= TOL


def test_bf16_rows_do_not_depend_on_the_call():
    """With bf16 weights every path of both kernels adds a column's products in one order, in every call: the same 40
    rows come out bit-identical from a call that the one-workgroup-per-tile kernel serves alone (one expert of 40
    rows) and from a call that launches both kernels, where they open an expert of 600 rows (persistent kernel), one
    of 150 (a single tile) and one of 300 (the first of two tiles side by side)."""
    from moe_gen_amd import ops
    h, I, r = 512, 768, 40
    g = torch.Generator().manual_seed(211)
    rows = torch.randn(r, h, generator=g).to(torch.bfloat16)
    one = make_experts(1, h, I, False, 212)[0]
    dm = [m.cuda() for m in one]
    small = ops.grouped_swiglu(rows.cuda(), None, ops.expert_pointers([dm[0]], [dm[1]], [dm[2]]),
                               torch.tensor([0, r], dtype=torch.int32).cuda(), r)
    counts = [600, 150, 300]
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    n = int(offsets[-1])
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    for e in range(3):
        x[offsets[e]:offsets[e] + r] = rows
    big = ops.grouped_swiglu(x.cuda(), None, ops.expert_pointers([dm[0]] * 3, [dm[1]] * 3, [dm[2]] * 3),
                             torch.from_numpy(offsets).cuda(), n)
    torch.cuda.synchronize()
    for e in range(3):
        assert torch.equal(big[offsets[e]:offsets[e] + r], small), f"expert of {counts[e]} rows"


@pytest.mark.parametrize("h,I", [(448, 512), (576, 640), (704, 384), (384, 448)])   # 7/8, 9/10, 11/6, 6/7 stages of 64 k
def test_bf16_weight_streamer_shapes_and_gather(h, I):
    """The bf16 weight streamer on every token-group count and both sides of each boundary, with stage counts that
    leave 0 ... 5 stages after its loop unrolled by six, rows gathered through row_map, and last N tiles that are
    ragged (down projection: h = 448, 576, 704 of 256 columns; gate/up: I = 448 of 128)."""
    counts = [16, 17, 32, 33, 48, 49, 64, 65, 80, 81, 96, 97, 112, 113, 128, 129, 144, 145, 160, 161, 176, 177, 192,
              1, 0, 15, 31, 47, 63] + [2] * 20
    print(f"bf16 streamer shapes h={h} I={I} counts={counts}", flush=True)
    y, ref32, refr = run_case(len(counts), h, I, counts, False, seed=161, use_row_map=True)
    assert np.isfinite(y).all()
    assert rel_max(y, ref32) <= TOL and rel_max(y, refr) <= TOL


@pytest.mark.parametrize("counts", [
    [129, 144, 145, 160, 176, 177, 192, 400, 600, 320, 449, 70],     # mean 255: both kernels; 400 = 256 + 144 left over
    [129, 150, 192, 170, 64, 65] + [5] * 20])                         # mean 35: the one-workgroup-per-tile kernel alone
@pytest.mark.parametrize("h,I", [(640, 384), (1024, 896)])            # 5 / 3 and 8 / 7 blocks of 128 k (odd and even counts)
def test_fp8_weight_streamer_tiles_of_129_to_192_rows(counts, h, I):
    """fp8 tiles of 129 to 192 rows -- experts of that size, and what the full 256-row tiles of a larger one leave over
    -- run on the streamer form with two weight buffers and 24 KiB of token rows per half.  Experts that share one set
    of weights and start with the same five rows: those rows come out bit-identical from every tile height, in the
    first list also from the persistent kernel (600 = 2 x 256 + 88 rows, 449 = 256 + 193) and the 128-row form (320 =
    256 + 64); the call gives the same bits every time, and the rows are within the layer bound of the oracle."""
    from moe_gen_amd import ops
    E = len(counts)
    print(f"fp8 streamer 129-192 h={h} I={I} counts={counts}", flush=True)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    n = int(offsets[-1])
    g = torch.Generator().manual_seed(297)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    for e in range(1, E):
        x[offsets[e]:offsets[e] + 5] = x[:5]
    one = make_experts(1, h, I, True, 298)[0]
    dm = [tuple(t.cuda() for t in m) for m in one]
    ptrs = ops.expert_pointers([dm[0][0]] * E, [dm[1][0]] * E, [dm[2][0]] * E, [dm[0][1]] * E, [dm[1][1]] * E, [dm[2][1]] * E)
    off_d = torch.from_numpy(offsets).cuda()
    xd = x.cuda()
    ys = [ops.grouped_swiglu(xd, None, ptrs, off_d, n).clone() for _ in range(6)]
    rm = torch.randperm(n, generator=g).to(torch.int32)
    xin = torch.empty_like(x)
    xin[rm.long()] = x
    y_map = ops.grouped_swiglu(xin.cuda(), rm.cuda(), ptrs, off_d, n)       # the same rows gathered through a row map
    torch.cuda.synchronize()
    for rep in range(1, 6):
        assert torch.equal(ys[rep], ys[0]), f"call {rep} differs from call 0"
    assert torch.equal(y_map, ys[0])
    alone = n // E < 128
    for e in range(1, E):
        if alone and counts[e] <= 64:
            continue        # (alone, up to 64 rows: the streamer form with its own order of summation)
        assert torch.equal(ys[0][offsets[e]:offsets[e] + 5], ys[0][:5]), f"expert {e} ({counts[e]} rows)"
    wg, wu, wd = (f32_of(m) for m in one)
    ref = O.mlp_f32(O.bf16_to_f32(bits(x)), wg, wu, wd)
    assert rel_max(O.bf16_to_f32(bits(ys[0])), ref) <= TOL


@pytest.mark.parametrize("h,I", [(512, 640), (640, 896), (896, 512)])      # 4 / 5 / 7 blocks of 128 k (gate/up), 5 / 7 / 4 (down)
def test_fp8_weight_streamer_shapes_and_gather(h, I):
    """The fp8 weight streamer on every token-group count and both sides of each boundary, with block counts that
    leave 0, 1 and 2 iterations after its loop unrolled by three, rows gathered through row_map, and a down
    projection whose last N tile is ragged (h = 640, 896)."""
    counts = [16, 17, 32, 33, 48, 49, 64, 1, 0, 15, 31, 47, 63]
    print(f"streamer shapes h={h} I={I} counts={counts}", flush=True)
    y, ref32, refr = run_case(len(counts), h, I, counts, True, seed=61, use_row_map=True)
    assert np.isfinite(y).all()
    assert rel_max(y, ref32) <= TOL and rel_max(y, refr) <= TOL


@pytest.mark.parametrize("fp8", [False, True])
def test_weight_streamer_row_outside_x_reads_zeros(fp8):
    """A row_map entry outside x is a row of zeros for the weight streamers too (their token DMA goes through a
    bounds-checked descriptor; such a row and the rows past an expert's last cost no memory request), and its
    neighbours are untouched: the other rows' bits equal those of a call with valid entries only."""
    from moe_gen_amd import ops
    E, h, I, per = 6, 512, 384, 20
    n = E * per
    mats = make_experts(E, h, I, fp8, 5)
    if fp8:
        dm = [[tuple(t.cuda() for t in m) for m in one] for one in mats]
        ptrs = ops.expert_pointers([o[0][0] for o in dm], [o[1][0] for o in dm], [o[2][0] for o in dm],
                                   [o[0][1] for o in dm], [o[1][1] for o in dm], [o[2][1] for o in dm])
    else:
        dm = [[m.cuda() for m in one] for one in mats]
        ptrs = ops.expert_pointers([o[0] for o in dm], [o[1] for o in dm], [o[2] for o in dm])
    x = torch.randn(n, h, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16).cuda()
    off = torch.arange(0, n + 1, per, dtype=torch.int32).cuda()
    rm = torch.arange(n, dtype=torch.int32)
    good = ops.grouped_swiglu(x, rm.cuda(), ptrs, off, n)
    bad = rm.clone()
    for r, v in ((7, n), (45, -1), (119, 2**31 - 1)):
        bad[r] = v
    got = ops.grouped_swiglu(x, bad.cuda(), ptrs, off, n)
    torch.cuda.synchronize()
    keep = torch.ones(n, dtype=torch.bool)
    keep[[7, 45, 119]] = False
    assert torch.equal(bits_t(got)[keep], bits_t(good)[keep])
    assert (got[~keep.cuda()].float() == 0).all()           # SwiGLU of a zero row is zero, and so is its down projection


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("E,mean", [(700, 3), (1024, 2), (600, 200), (400, 200)])
def test_grouped_many_experts(fp8, E, mean):
    """More experts than threads in a workgroup (the M-tile prefix scan takes two passes), up to the
    maximum of 1024, with empty experts sprinkled in; the last two cases have about 200 rows per expert (400
    experts: the persistent kernel with its per-expert tables in LDS; 600: one workgroup per tile, two
    128-row tiles for most experts)."""
    print(f"grouped many experts fp8={fp8} E={E} mean={mean}", flush=True)
    rng = np.random.default_rng(E)
    counts = rng.poisson(mean, E)
    counts[::7] = 0
    y, ref32, _ = run_case(E, 128, 128, counts, fp8, seed=5)
    assert np.isfinite(y).all() and rel_max(y, ref32) <= TOL


def test_grouped_too_many_experts_is_an_error():
    from moe_gen_amd import ops
    E = 1025
    w = torch.zeros(128, 128, dtype=torch.bfloat16, device="cuda")
    ptrs = ops.expert_pointers([w] * E, [w] * E, [w] * E)
    off = torch.zeros(E + 1, dtype=torch.int32, device="cuda")
    off[1:] = 4
    x = torch.zeros(4, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="n_experts"):
        ops.grouped_swiglu(x, None, ptrs, off, 4)


@pytest.mark.parametrize("fp8", [False, True])
def test_grouped_more_tiles_than_cus(fp8):
    """808 gate/up tiles and 404 down tiles of 256 rows on 256 CUs: with fp8 weights every persistent
    workgroup hands its pipeline over from tile to tile (different experts, a ragged last tile, a
    10-row expert in between); rows are gathered through a row map."""
    print(f"grouped more tiles than CUs fp8={fp8}", flush=True)
    y, ref32, _ = run_case(4, 1024, 1024, [9000, 7000, 10, 9000], fp8, seed=31, use_row_map=True)
    assert np.isfinite(y).all()
    err = rel_max(y, ref32)
    print(f"  max-rel vs fp32 {err:.3e}", flush=True)
    assert err <= TOL


@pytest.mark.parametrize("fp8", [False, True])
def test_grouped_swiglu_row_map(fp8):
    y, ref32, _ = run_case(4, 256, 256, [100, 0, 300, 77], fp8, seed=23, use_row_map=True)
    assert rel_max(y, ref32) <= TOL


def _one_expert(h, I, seed):
    from moe_gen_amd import ops
    g = torch.Generator().manual_seed(seed)
    ws = [(torch.randn(shape, generator=g) * 0.05).to(torch.bfloat16) for shape in ((I, h), (I, h), (h, I))]
    ptrs = ops.expert_pointers(*[[w.cuda()] for w in ws])
    return ws, ptrs


@pytest.mark.parametrize("h,I,n", [(256, 256, 600), (256, 8192, 1100), (192, 256, 600), (256, 256, 100)])
def test_row_map_entry_outside_x_reads_zeros(h, I, n):
    """A row_map entry beyond x_rows stands for a row of zeros (no fault), and every other row is unaffected: the
    persistent kernel fetches gathered rows through a buffer descriptor that ends with x (1100 rows x 64 N tiles:
    a round of its tiles and more), the other kernel checks the entry (600 rows: six tiles, the persistent kernel's
    short last round as half tiles; K = 192 and 100 rows: calls it serves alone)."""
    from moe_gen_amd import ops
    ws, ptrs = _one_expert(h, I, 41)
    g = torch.Generator().manual_seed(42)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    rm = torch.randperm(n, generator=g).to(torch.int32)
    bad = [3, n // 2 + 7, n - 1]
    rm_bad = rm.clone()
    rm_bad[bad] = torch.tensor([n, n + 5, 2 ** 20], dtype=torch.int32)
    off = torch.tensor([0, n], dtype=torch.int32, device="cuda")
    y_ok = ops.grouped_swiglu(x.cuda(), rm.cuda(), ptrs, off, n)
    y_bad = ops.grouped_swiglu(x.cuda(), rm_bad.cuda(), ptrs, off, n)
    torch.cuda.synchronize()
    keep = np.ones(n, bool)
    keep[bad] = False
    assert np.array_equal(bits(y_ok)[keep], bits(y_bad)[keep])
    assert (y_bad[bad].float().cpu().numpy() == 0).all()        # silu(0) * 0 through the down projection


@pytest.mark.parametrize("fp8", [False, True])
def test_gathered_rows_of_an_input_beyond_4_gib(fp8):
    """Gathered rows are addressed with 32-bit byte offsets only while x is smaller than 4 GiB; a larger
    x takes the one-workgroup-per-tile kernel with 64-bit addresses (with fp8 weights its register-staged body: the
    weight streamers address rows through a 32-bit descriptor).  The rows used sit at both ends of x."""
    from moe_gen_amd import ops
    h, I, n = 2048, 256, 512
    x_rows = (1 << 32) // (h * 2) + 4096                          # 4 GiB + 16 MiB of bf16 rows
    if fp8:
        mats = make_experts(1, h, I, True, 43)[0]
        dm = [tuple(t.cuda() for t in m) for m in mats]
        ptrs = ops.expert_pointers([dm[0][0]], [dm[1][0]], [dm[2][0]], [dm[0][1]], [dm[1][1]], [dm[2][1]])
        wg, wu, wd = (f32_of(m) for m in mats)
    else:
        ws, ptrs = _one_expert(h, I, 43)
        wg, wu, wd = (O.bf16_to_f32(bits(w)) for w in ws)
    g = torch.Generator().manual_seed(44)
    rows = torch.randn(n, h, generator=g).to(torch.bfloat16)
    x = torch.zeros(x_rows, h, dtype=torch.bfloat16, device="cuda")
    where = torch.cat([torch.arange(n // 2), torch.arange(x_rows - n // 2, x_rows)]).to(torch.int32)
    where = where[torch.randperm(n, generator=g)]
    x[where.long().cuda()] = rows.cuda()
    off = torch.tensor([0, n], dtype=torch.int32, device="cuda")
    y = ops.grouped_swiglu(x, where.cuda(), ptrs, off, n)
    y_ref = ops.grouped_swiglu(rows.cuda(), None, ptrs, off, n)   # the same rows, sorted: the persistent kernel
    torch.cuda.synchronize()
    del x
    ref32 = O.mlp_f32(O.bf16_to_f32(bits(rows)), wg, wu, wd)
    assert rel_max(O.bf16_to_f32(bits(y)), ref32) <= TOL
    assert rel_max(O.bf16_to_f32(bits(y_ref)), ref32) <= TOL


def test_gathered_rows_beyond_4_gib_at_every_tile_kind_bf16():
    """The register-staged body behind the bf16 weight streamer (4 GiB of gathered rows or more) takes what the
    streamer takes: single tiles of up to 192 rows (above 128 as two passes of 128 rows), the halves of an expert of
    257 to 384 rows, 128-row slices.  Experts that share one set of weights, rows gathered from both ends of a 4 GiB
    x: every row equals, bit for bit, what the same rows give sorted and through the streamer (one order of
    summation for every bf16 path)."""
    from moe_gen_amd import ops
    h, I = 2048, 256
    counts = [150, 192, 300, 40, 129, 70, 384, 500]
    E, n = len(counts), sum(counts)
    x_rows = (1 << 32) // (h * 2) + 4096                          # 4 GiB + 16 MiB of bf16 rows
    ws, _ = _one_expert(h, I, 47)
    dw = [w.cuda() for w in ws]
    ptrs = ops.expert_pointers([dw[0]] * E, [dw[1]] * E, [dw[2]] * E)
    g = torch.Generator().manual_seed(48)
    rows = torch.randn(n, h, generator=g).to(torch.bfloat16)
    x = torch.zeros(x_rows, h, dtype=torch.bfloat16, device="cuda")
    where = torch.cat([torch.arange(n // 2), torch.arange(x_rows - (n - n // 2), x_rows)]).to(torch.int32)
    where = where[torch.randperm(n, generator=g)]
    x[where.long().cuda()] = rows.cuda()
    off = torch.tensor(np.concatenate([[0], np.cumsum(counts)]), dtype=torch.int32, device="cuda")
    print(f"4 GiB gather, bf16, counts={counts}", flush=True)
    y = ops.grouped_swiglu(x, where.cuda(), ptrs, off, n)
    y_ref = ops.grouped_swiglu(rows.cuda(), None, ptrs, off, n)
    torch.cuda.synchronize()
    del x
    wg, wu, wd = (O.bf16_to_f32(bits(w)) for w in ws)
    assert rel_max(O.bf16_to_f32(bits(y_ref)), O.mlp_f32(O.bf16_to_f32(bits(rows)), wg, wu, wd)) <= TOL
    assert torch.equal(y, y_ref)


@pytest.mark.parametrize("fp8", [False, True])
def test_expert_sub_range_through_the_persistent_kernel(fp8):
    """A call on experts [1, 3) of four with absolute row offsets (weights handed out in waves): the rows
    of the other experts stay untouched, the range's rows match the call on all experts."""
    from moe_gen_amd import ops
    E, h, I = 4, 256, 256
    counts = np.array([300, 520, 260, 290], np.int32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    n = int(offsets[-1])
    g = torch.Generator().manual_seed(47)
    x = torch.randn(n, h, generator=g).to(torch.bfloat16).cuda()
    mats = make_experts(E, h, I, fp8, 48)
    dev = lambda m: tuple(t.cuda() for t in m) if isinstance(m, tuple) else m.cuda()
    dm = [[dev(m) for m in one] for one in mats]

    def pointers(sel):
        if fp8:
            return ops.expert_pointers([dm[e][0][0] for e in sel], [dm[e][1][0] for e in sel], [dm[e][2][0] for e in sel],
                                       [dm[e][0][1] for e in sel], [dm[e][1][1] for e in sel], [dm[e][2][1] for e in sel])
        return ops.expert_pointers([dm[e][0] for e in sel], [dm[e][1] for e in sel], [dm[e][2] for e in sel])

    off_d = torch.from_numpy(offsets).cuda()
    y_all = ops.grouped_swiglu(x, None, pointers(range(E)), off_d, n)
    act = torch.zeros(n, I, dtype=torch.bfloat16, device="cuda")
    y = torch.full((n, h), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.grouped_swiglu(x, None, pointers([1, 2]), off_d[1:4].contiguous(), n, act, y,
                       rows_bound=int(offsets[3] - offsets[1]))
    torch.cuda.synchronize()
    a, b = int(offsets[1]), int(offsets[3])
    assert torch.equal(y[a:b], y_all[a:b])
    assert (y[:a] == 7.0).all() and (y[b:] == 7.0).all()


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("E,h,I,counts", [
    (2, 128, 128, [300, 260]),                # two k-stages: the shortest pipeline the persistent kernel runs
    (2, 128, 384, [513, 256]),                # gate/up: 2 stages; down: 6; a tile of one row
    (3, 256, 128, [700, 0, 300]),             # down projection with 2 stages, an empty expert in between
    (512, 128, 128, [200] * 512),             # as many experts as the kernel keeps tables for
])
def test_persistent_kernel_corner_shapes(fp8, E, h, I, counts):
    """The 256-row persistent kernel (experts above 192 rows, K a multiple of 128) at the ends of what
    it accepts; rows gathered through a row map."""
    print(f"persistent corners fp8={fp8} E={E} h={h} I={I}", flush=True)
    y, ref32, _ = run_case(E, h, I, counts, fp8, seed=37, use_row_map=True)
    assert np.isfinite(y).all() and rel_max(y, ref32) <= TOL


EDGE_COUNTS = [0, 1, 17, 64, 65, 128, 129, 144, 145, 160, 161, 192, 193, 256, 257, 300, 384, 385, 449, 700]


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("seed", range(10))
def test_grouped_seeded_mixtures(fp8, seed):
    """Seeded draws of expert count, sizes and per-expert rows from both sides of every tile-height and
    kernel boundary (64 / 128 / 144 / 160 / 192 / 256 / 384 rows), with and without a row map: whichever
    kernels and tile forms the launcher picks for the mixture, every row matches the oracle, and a second
    call returns the same bits."""
    rng = np.random.default_rng(1000 + seed)
    E = int(rng.choice([1, 2, 3, 5, 8, 13]))
    h, I = 128 * int(rng.integers(1, 6)), 128 * int(rng.integers(1, 6))
    kind = ["few", "middle", "edges", "many"][seed % 4]
    counts = {"few": rng.integers(0, 70, E), "middle": rng.integers(100, 400, E),
              "edges": rng.choice(EDGE_COUNTS, E), "many": rng.integers(300, 900, E)}[kind]
    counts = [int(c) for c in counts]
    if sum(counts) == 0:
        counts[0] = 33
    use_map = bool(rng.integers(0, 2))
    print(f"mixture fp8={fp8} seed={seed} E={E} h={h} I={I} {kind} row_map={use_map} counts={counts}", flush=True)
    y, ref32, refr = run_case(E, h, I, counts, fp8, seed=300 + seed, use_row_map=use_map)
    y2, _, _ = run_case(E, h, I, counts, fp8, seed=300 + seed, use_row_map=use_map)
    assert np.isfinite(y).all()
    assert rel_max(y, ref32) <= TOL and rel_max(y, refr) <= TOL
    assert np.array_equal(y, y2)


@pytest.mark.parametrize("n_src,n", [(300, 600), (60, 120)])
def test_row_map_may_repeat_rows(n_src, n):
    """Several sorted rows may name the same source row (a token routed to k experts).  Both launches of a case
    run the same kernel (the persistent kernel / one workgroup per tile): the two walk k from different stages
    and may differ in the last bit."""
    from moe_gen_amd import ops
    h, I = 256, 256
    ws, ptrs = _one_expert(h, I, 51)
    g = torch.Generator().manual_seed(52)
    x = torch.randn(n_src, h, generator=g).to(torch.bfloat16)
    rm = torch.randint(0, n_src, (n,), generator=g, dtype=torch.int32)
    off = torch.tensor([0, n], dtype=torch.int32, device="cuda")
    y = ops.grouped_swiglu(x.cuda(), rm.cuda(), ptrs, off, n)
    y_src = ops.grouped_swiglu(x.cuda(), None, ptrs, torch.tensor([0, n_src], dtype=torch.int32, device="cuda"), n_src)
    torch.cuda.synchronize()
    wg, wu, wd = (O.bf16_to_f32(bits(w)) for w in ws)
    ref32 = O.mlp_f32(O.bf16_to_f32(bits(x)), wg, wu, wd)[rm.long().numpy()]
    assert rel_max(O.bf16_to_f32(bits(y)), ref32) <= TOL
    assert np.array_equal(bits(y), bits(y_src)[rm.long().numpy()])       # a row's result does not depend on its tile


def test_grouped_single_expert_is_plain_mlp():
    """E = 1 reduces to a dense SwiGLU MLP: compare with torch's own bf16 linear layers on the GPU."""
    from moe_gen_amd import DeepseekV3Config, DeepseekV3MLP
    cfg = DeepseekV3Config(hidden_size=512, intermediate_size=768)
    mlp = DeepseekV3MLP(cfg).cuda().to(torch.bfloat16)
    x = torch.randn(3, 70, 512, device="cuda").to(torch.bfloat16)
    y = mlp(x)
    F = torch.nn.functional
    with torch.no_grad():
        ref = F.linear(F.silu(F.linear(x, mlp.gate_proj.weight)) * F.linear(x, mlp.up_proj.weight), mlp.down_proj.weight)
    assert rel_max(y.float().cpu().numpy(), ref.float().cpu().numpy()) <= TOL


@pytest.mark.parametrize("rows,cols", [(128, 128), (130, 200), (1, 16), (257, 1000), (2048, 7168)])
def test_dequant_bit_exact(rows, cols):
    from moe_gen_amd import ops
    g = torch.Generator().manual_seed(rows * 31 + cols)
    q = torch.randint(0, 256, (rows, cols), generator=g, dtype=torch.uint8)
    q[(q & 0x7F) == 0x7F] = 0                   # NaN patterns carry no ordering of payload bits
    s = torch.rand((-(-rows // 128), -(-cols // 128)), generator=g) * 0.01 + 1e-4
    out = ops.dequant_fp8_block128(q.cuda().view(torch.float8_e4m3fn), s.cuda())
    torch.cuda.synchronize()
    ref = O.dequant_block(q.numpy(), s.numpy())
    assert np.array_equal(bits(out), ref)


def test_fp8_decode_table_on_device():
    """All 256 byte values with scale 1: the device conversion is OCP e4m3fn (max 448, no inf)."""
    from moe_gen_amd import ops
    q = torch.arange(256, dtype=torch.uint8).repeat(16).view(16, 256)
    s = torch.ones((1, 2))
    out = ops.dequant_fp8_block128(q.cuda().view(torch.float8_e4m3fn), s.cuda()).float().cpu().numpy()[0]
    tab = O.fp8_table()
    ok = ~np.isnan(tab)
    assert np.array_equal(out[ok], tab[ok]) and np.isnan(out[~ok]).all()


def test_dequant_golden_fixture():
    import os
    from moe_gen_amd import ops
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "fp8_dequant.npz"))
    out = ops.dequant_fp8_block128(torch.from_numpy(z["q"]).cuda().view(torch.float8_e4m3fn), torch.from_numpy(z["scale"]).cuda())
    assert np.array_equal(bits(out), z["out"])


@pytest.mark.parametrize("fp8", [False, True])
def test_swiglu_epilogue_alone(fp8):
    """The SiLU*mul epilogue pinned on its own: one-hot token rows make every gate and up output a
    single exact product, g[r,c] = Wg[c, r], u[r,c] = Wu[c, r], so `act` (the gate/up launch's
    output) must be bf16(bf16(silu(g)) * u) -- torch's own bf16 silu and bf16 mul on the CPU are the
    witness.  The kernel evaluates silu with the hardware exp and reciprocal (about 1e-6 relative),
    so bf16(silu(g)) may land on the other side of a rounding boundary on a few elements: one bf16
    step there, which the product with u turns into at most two steps of the result (a factor at the
    bottom of its binade, a product at the top of one).  A swapped gate/up role, a missing rounding
    point or a wrong sign fails everywhere."""
    from moe_gen_amd import ops
    from moe_gen_amd.synthetic import quantize_fp8_block128
    h = I = 128
    n = 3 * h                                            # every one-hot row three times, with different scales
    g = torch.Generator().manual_seed(17)
    if fp8:                                              # exactly representable after block quantisation: powers of two times small integers
        wg = (torch.randint(-12, 13, (I, h), generator=g).float() * 0.25)
        wu = (torch.randint(-8, 9, (I, h), generator=g).float() * 0.5)
        wg[0, 0], wu[0, 0] = 28.0, 14.0                 # fixes each block's scale: amax = 28 -> 28/448 = 2^-4, 14/448 = 2^-5
        qg, qu = quantize_fp8_block128(wg), quantize_fp8_block128(wu)
        wg_f = torch.from_numpy(O.bf16_to_f32(O.dequant_block(bits(qg[0]), qg[1].numpy())))
        wu_f = torch.from_numpy(O.bf16_to_f32(O.dequant_block(bits(qu[0]), qu[1].numpy())))
        assert torch.equal(wg_f, wg) and torch.equal(wu_f, wu)
        qd = quantize_fp8_block128(torch.zeros(h, I))
        ptrs = ops.expert_pointers([qg[0].cuda()], [qu[0].cuda()], [qd[0].cuda()], [qg[1].cuda()], [qu[1].cuda()], [qd[1].cuda()])
    else:
        wg = (torch.randn(I, h, generator=g) * 4).to(torch.bfloat16)
        wu = (torch.randn(I, h, generator=g) * 2).to(torch.bfloat16)
        wg_f, wu_f = wg.float(), wu.float()
        ptrs = ops.expert_pointers([wg.cuda()], [wu.cuda()], [torch.zeros(h, I, dtype=torch.bfloat16).cuda()])
    scales = torch.tensor([1.0, 0.5, 4.0])
    x = torch.zeros(n, h, dtype=torch.bfloat16)
    for r in range(n):
        x[r, r % h] = scales[r // h]
    act = torch.empty(n, I, dtype=torch.bfloat16, device="cuda")
    y = torch.empty(n, h, dtype=torch.bfloat16, device="cuda")
    off = torch.tensor([0, n], dtype=torch.int32, device="cuda")
    ops.grouped_swiglu(x.cuda(), None, ptrs, off, n, act, y, ops.PHASE_GATE_UP)
    torch.cuda.synchronize()
    gate = torch.stack([wg_f[:, r % h] * scales[r // h] for r in range(n)]).to(torch.bfloat16)   # exact: one product
    up = torch.stack([wu_f[:, r % h] * scales[r // h] for r in range(n)]).to(torch.bfloat16)
    want = torch.nn.functional.silu(gate) * up                                                    # bf16 modules, as the reference
    got_bits, want_bits = bits(act).astype(np.int32), bits(want).astype(np.int32)
    diff = np.abs(got_bits - want_bits)
    assert diff.max() <= 2, f"epilogue off by {diff.max()} bf16 steps"
    assert (diff > 0).mean() < 0.01, f"{(diff > 0).mean():.2%} of the elements differ"
    assert (diff > 1).mean() < 0.001, f"{(diff > 1).mean():.3%} of the elements differ by two steps"
