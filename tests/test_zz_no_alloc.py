"""moe_dispatch_static -- the entry point that allocates nothing (its per-segment counters live in
a device array built into the library) -- against moe_dispatch, through the C ABI, bit for bit."""
import numpy as np
import pytest
import torch

from moe_gen_amd import _native as N


def _run(entry, idx, E, x=None):
    """Call `entry` ("moe_dispatch" or "moe_dispatch_static") on device tensors allocated here."""
    n, k = idx.shape
    dev = idx.device
    i32 = dict(dtype=torch.int32, device=dev)
    counts, offsets = torch.full((E,), -7, **i32), torch.full((E + 1,), -7, **i32)
    perm, pos, row_map = (torch.full((n * k,), -7, **i32) for _ in range(3))
    h = 0 if x is None else x.shape[1]
    xs = None if x is None else torch.zeros((n * k, h), dtype=torch.bfloat16, device=dev)
    p = lambda t: None if t is None else t.data_ptr()
    st = torch.cuda.current_stream().cuda_stream
    L = N.lib()
    if entry == "moe_dispatch":
        wsb = L.moe_dispatch_workspace_bytes(n, k, E)
        ws = torch.empty(wsb, dtype=torch.uint8, device=dev)
        rc = L.moe_dispatch(p(idx), n, k, E, p(counts), p(offsets), p(perm), p(pos), p(row_map), p(x), h, p(xs), p(ws), wsb, st)
    else:
        rc = L.moe_dispatch_static(p(idx), n, k, E, p(counts), p(offsets), p(perm), p(pos), p(row_map), p(x), h, p(xs), st)
    N.check(rc, entry)
    torch.cuda.synchronize()
    return counts, offsets, perm, pos, row_map, xs


def _idx(n, k, E, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.rand((n, E), generator=g, device="cuda").topk(k, dim=1).indices.to(torch.int32)


@pytest.mark.gpu
def test_static_dispatch_matches_dispatch_on_consecutive_calls():
    """Two calls in a row share the built-in array; the second is smaller (fewer segments, fewer
    experts) and must not see what the first left behind.  Then the DeepSeek-V3 workload size."""
    print("no-alloc dispatch: 40000x8/256, then 3000x6/64, then 65536x8/256", flush=True)
    for n, k, E, h, seed in ((40000, 8, 256, 64, 1), (3000, 6, 64, 128, 2), (65536, 8, 256, 0, 3), (1, 1, 1, 8, 4)):
        idx = _idx(n, k, E, seed)
        x = torch.randn(n, h, device="cuda").to(torch.bfloat16) if h else None
        want = _run("moe_dispatch", idx, E, x)
        got = _run("moe_dispatch_static", idx, E, x)
        for name, a, b in zip(("counts", "offsets", "perm", "pos", "row_map", "xs"), want, got):
            if a is None:
                assert b is None
                continue
            assert torch.equal(a.view(torch.int16) if a.dtype == torch.bfloat16 else a,
                               b.view(torch.int16) if b.dtype == torch.bfloat16 else b), (n, k, E, name)
        assert torch.equal(got[2].long(), torch.argsort(idx.view(-1).long(), stable=True))
    # empty input: counts and offsets are zeroed, nothing else is touched
    e = torch.zeros((0, 4), dtype=torch.int32, device="cuda")
    got = _run("moe_dispatch_static", e, 16)
    assert got[0].sum().item() == 0 and got[1].sum().item() == 0


@pytest.mark.gpu
def test_static_dispatch_captured_in_a_graph():
    """The use the entry point is documented for: after one eager call on the device (which looks the array's
    address up), further calls are captured into a HIP graph -- three kernel launches, no allocation, no memset --
    and every replay, with the program's own eager work and synchronisations in between and with new routing in the
    same buffers, gives what moe_dispatch gives eagerly."""
    n, k, E = 5000, 6, 160
    print(f"no-alloc dispatch under graph capture: {n}x{k}/{E}", flush=True)
    L = N.lib()
    idx_static = _idx(n, k, E, 11)
    _run("moe_dispatch_static", idx_static, E)                       # eager: resolves the symbol address on this device
    i32 = dict(dtype=torch.int32, device="cuda")
    counts, offsets = torch.zeros(E, **i32), torch.zeros(E + 1, **i32)
    perm, pos, row_map = (torch.zeros(n * k, **i32) for _ in range(3))
    p = lambda t: t.data_ptr()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                                    # warm-up on the side stream, as torch asks before a capture
        N.check(L.moe_dispatch_static(p(idx_static), n, k, E, p(counts), p(offsets), p(perm), p(pos), p(row_map), None, 0, None,
                                      side.cuda_stream), "moe_dispatch_static")
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = L.moe_dispatch_static(p(idx_static), n, k, E, p(counts), p(offsets), p(perm), p(pos), p(row_map), None, 0, None,
                                   torch.cuda.current_stream().cuda_stream)
    N.check(rc, "moe_dispatch_static under capture")
    torch.cuda.synchronize()
    for it in range(4):
        idx_static.copy_(_idx(n, k, E, 20 + it))                     # new routing in the captured buffers
        for t in (counts, offsets, perm, pos, row_map):
            t.fill_(-3)
        graph.replay()
        torch.cuda.synchronize()
        want = _run("moe_dispatch", idx_static, E)                    # eager work of the program between the replays
        for name, a, b in zip(("counts", "offsets", "perm", "pos", "row_map"), want, (counts, offsets, perm, pos, row_map)):
            assert torch.equal(a, b), (it, name)


def test_static_dispatch_rejects_what_does_not_fit():
    """Size and argument checks happen on the host, before anything touches a device."""
    L = N.lib()
    big_n = 2 ** 21 // 8 + 2048                                      # one segment more than fits with 256 experts
    rc = L.moe_dispatch_static(1, big_n, 8, 256, 1, 1, 1, 1, None, None, 0, None, None)
    assert rc == -2 and "exceed the built-in scratch" in N.last_error() and "moe_dispatch" in N.last_error()
    assert L.moe_dispatch_static(1, 4, 2, 300, 1, 1, 1, 1, None, None, 0, None, None) == -1
    assert L.moe_dispatch_static(1, 4, 2, 8, None, 1, 1, 1, None, None, 0, None, None) == -1
