"""Weight staging on the device: pinned host -> HBM slots on the copy stream, event hand-off."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_stager_roundtrip_and_reuse():
    from moe_gen_amd import Stager
    shapes = {"routed_expert": {"gate_proj.weight": ((64, 128), torch.bfloat16),
                                "up_proj.weight": ((64, 128), torch.bfloat16),
                                "down_proj.weight": ((128, 64), torch.bfloat16)}}
    st = Stager(shapes, {"routed_expert": 3}, model_type="deepseek_v2", num_hidden_layers=4, num_local_experts=8)
    host = {}
    for L in (2, 3):
        for e in range(8):
            t = {k: torch.randn(s, dtype=torch.float32).to(d).pin_memory() for k, (s, d) in shapes["routed_expert"].items()}
            host[(L, e)] = t
            st.add_module(f"routed_expert_{L}_{e}", "routed_expert", t)
    for L in (2, 3):
        for e in range(8):
            st.clear_expert_buffer(L, e)
            if e % 3 == 1:
                continue                       # a skipped expert: reclaimed later by clear_expert_buffer
            w = st.get_weights(f"routed_expert_{L}_{e}")
            for k, v in w.items():
                assert torch.equal(v.cpu(), host[(L, e)][k]), (L, e, k)
            st.free_weights_buffer(f"routed_expert_{L}_{e}")
    st.sync()
    copies, nbytes = st.stats()
    assert copies >= 16 and nbytes == copies * 3 * 64 * 128 * 2
    with pytest.raises(RuntimeError):
        st.get_weights("routed_expert_9_9")
    st.close()


def test_stager_overlaps_with_compute():
    """A copy issued before a long kernel on the compute stream completes without waiting for it."""
    from moe_gen_amd import Stager
    shapes = {"routed_expert": {"w": ((4096, 4096), torch.bfloat16)}}
    st = Stager(shapes, {"routed_expert": 2})
    src = [torch.randn(4096, 4096).to(torch.bfloat16).pin_memory() for _ in range(4)]
    for i, t in enumerate(src):
        st.add_module(f"routed_expert_0_{i}", "routed_expert", {"w": t})
    a = torch.randn(4096, 4096, device="cuda")
    for i in range(4):
        w = st.get_weights(f"routed_expert_0_{i}")["w"]
        s = (w.float() @ a).sum()               # compute on the current stream reads the slot
        same = torch.equal(w, src[i].cuda())    # enqueued before the slot is let go
        st.free_weights_buffer(f"routed_expert_0_{i}")
        assert torch.isfinite(s) and same
    torch.cuda.synchronize()
    st.close()


def check_against_oracle(blk_resident, w, x_cpu, out, blk_run):
    """Routing bit-exact and output within the layer bound (2e-2 of the fp32 oracle), as in
    test_gpu_layer.py; `blk_resident` still owns the weights the oracle reads."""
    import numpy as np
    from oracle import oracle as O
    from util import bits, oracle_spec, oracle_weights, rel_max
    mode = {"v3": O.COMBINE_F32, "v2": O.COMBINE_BF16_PROD, "mixtral": O.COMBINE_BF16_SEQ}[w.family]
    ref32, aux = O.layer(bits(x_cpu).reshape(w.n, w.h), oracle_weights(blk_resident, w.family), oracle_spec(w), mode,
                         rounding="f32")
    assert np.array_equal(blk_run.last_topk_idx.cpu().numpy(), aux["idx"])
    assert np.array_equal(blk_run.last_counts.cpu().numpy(), aux["counts"])
    err = rel_max(O.bf16_to_f32(bits(out)).reshape(w.n, w.h), ref32)
    assert err <= 2e-2, err


class FakeCoreEngine:
    """Stands in for MoE-Gen's pybind `core_engine` (MoE_Gen_Binding.cpp:45-65) with the reference's
    slot semantics: a pool of `n_slots` device buffers per module type that a copy worker fills in
    registration order whenever a slot is free (HtoD_Engine.cpp:201-268), a get_weights that can
    only return what the worker delivered (GPU_Weight_Buffer.cpp:171-246; the reference spins, this
    one raises), and a free_weights_buffer that lets the worker overwrite the slot AT ONCE
    (GPU_Weight_Buffer.cpp:163-169) -- so a caller that frees while its kernels still read the slot
    gets the next module's weights in its output."""

    def __init__(self, weights, n_slots):
        self.src = weights                                   # key -> {tensor name -> device tensor}
        self.queue = {"routed_expert": [k for k in weights if k.startswith("routed")],
                      "shared_expert": [k for k in weights if k.startswith("shared")]}
        self.n_slots = dict(n_slots)
        self.slots = {t: [None] * n for t, n in self.n_slots.items()}
        self.mem = {t: [None] * n for t, n in self.n_slots.items()}
        self.held, self.calls, self.max_held = set(), [], 0
        self.side = torch.cuda.Stream()

    @staticmethod
    def _type(key):
        return "routed_expert" if key.startswith("routed") else "shared_expert"

    def _pump(self):
        for t, q in self.queue.items():
            while q and None in self.slots[t] and q[0] not in self.slots[t]:
                s = self.slots[t].index(None)
                key = q.pop(0); q.append(key)
                if self.mem[t][s] is None:
                    self.mem[t][s] = {n: torch.empty_like(v) for n, v in self.src[key].items()}
                with torch.cuda.stream(self.side):          # the worker's own stream, then a host wait
                    for n, v in self.src[key].items():
                        self.mem[t][s][n].copy_(v)
                self.side.synchronize()
                self.slots[t][s] = key

    def get_weights(self, key):
        self._pump()
        t = self._type(key)
        if key not in self.slots[t]:
            raise RuntimeError(f"get_weights({key}) would block forever: the pool holds {self.slots[t]}")
        self.held.add(key); self.max_held = max(self.max_held, len(self.held))
        self.calls.append(("get", key))
        return self.mem[t][self.slots[t].index(key)]

    def free_weights_buffer(self, key):
        self.calls.append(("free", key)); self.held.remove(key)
        t = self._type(key)
        self.slots[t][self.slots[t].index(key)] = None
        self._pump()                                         # the worker refills the slot immediately

    def clear_expert_buffer(self, layer_idx, expert_idx):
        self.calls.append(("clear", layer_idx, expert_idx))


class ExpertWrapperLike(torch.nn.Module):
    """Attribute-for-attribute what the reference's Expert_Wrapper exposes (Wrapper.py:437-468)."""
    phase = "prefill"

    def __init__(self, module, layer_idx, expert_idx, core_engine, scales, engine_config):
        super().__init__()
        self.module, self.layer_idx, self.expert_idx = module, layer_idx, expert_idx
        self.core_engine, self.get_weights, self.weight_dequant_scale = core_engine, True, scales
        self.engine_config = engine_config
        self.expert_weights_idx = (f"routed_expert_{layer_idx}_{expert_idx}" if expert_idx >= 0
                                   else f"shared_expert_{layer_idx}")


@pytest.mark.parametrize("name,n_slots,phase,resident", [
    ("deepseek_v3_w8a16", 20, "prefill", ()), ("deepseek_v2_236b", 20, "prefill", ()), ("deepseek_v3_w8a16", 256, "prefill", ()),
    ("deepseek_v2_236b", 7, "prefill", ()),
    ("mixtral_8x7b", 8, "prefill", ()), ("mixtral_8x7b", 3, "prefill", ()),           # pool = E and pool < E
    ("deepseek_v3_w8a16", 20, "decoding", ()), ("mixtral_8x7b", 3, "decoding", ()),  # the decoding pool is the one that counts
    ("deepseek_v2_236b", 7, "prefill", (0, 5, 6, 159)), ("mixtral_8x7b", 3, "prefill", (2, 7)),   # some experts stay resident
])
def test_block_with_engine_backed_experts(name, n_slots, phase, resident):
    """The block fed through MoE-Gen's expert-wrapper protocol against an engine with the
    reference's default pool of 20 routed-expert slots (deepseekv3_initializer.py:912-916), far
    fewer than the layer's experts: same bits as with resident weights, parity with the oracle,
    never more than the pool held, one get/free per expert.  Mixtral's experts are wrapped the same
    way (Mixtral_Initializer.py:761-787; w1 / w3 / w2, no shared expert).  In the decoding phase
    (Expert_Wrapper.phase == "decoding", Wrapper.py:434) the pool size is read from
    num_decoding_module_buffer (deepseekv3_initializer.py:918-927): the engine here then has that many
    slots and a prefill entry that would be wrong.  `resident`: experts the initializer left out of the
    copy task keep their weights and get_weights = False (deepseekv3_initializer.py:1259-1266)."""
    from types import SimpleNamespace as NS
    from moe_gen_amd import synthetic
    w = synthetic.WORKLOADS[name].scaled(n=256, h=512, I=256, seq=64)
    print(f"engine-backed {name} pool {n_slots} of {w.E} experts, phase {phase}, resident {resident}", flush=True)
    blk = synthetic.build_block(w, device="cuda", gen_device="cpu")
    x_cpu = synthetic.hidden_states(w, "cpu")
    x = x_cpu.cuda()
    first = lambda o: o[0] if isinstance(o, tuple) else o
    # (the staged walk cannot run the shared expert as a group of the routed call, and with fp8 weights that changes
    # the order its products are added in: the resident reference keeps the two calls apart too)
    blk.join_shared = False
    ref = first(blk(x)).clone()
    resident_blk = synthetic.build_block(w, device="cuda", gen_device="cpu")     # keeps the weights for the oracle
    names = blk.experts[0].names
    has_shared = w.family != "mixtral"
    L = 7
    weights, wrapped = {}, []

    def detach(mlp, key):
        weights[key] = {f"{n}.weight": getattr(mlp, n).weight.data.clone() for n in names}
        scales = {f"{n}.weight_scale_inv": getattr(mlp, n).weight_scale_inv.data for n in names} if w.fp8 else None
        for n in names:                                   # placeholders, as MoE-Gen leaves them
            getattr(mlp, n).weight.data = torch.zeros(1, dtype=torch.bfloat16, device="cuda")
        return scales

    scales = [None if e in resident else detach(ex, f"routed_expert_{L}_{e}") for e, ex in enumerate(blk.experts)]
    sscale = detach(blk.shared_experts, f"shared_expert_{L}") if has_shared else None
    eng = FakeCoreEngine(weights, {"routed_expert": n_slots, "shared_expert": 1})
    in_phase = {"routed_expert": n_slots, "shared_expert": 1}
    other = {"routed_expert": 4 * n_slots if phase == "prefill" else 1, "shared_expert": 1}
    cfg = NS(GPU_Buffer_Config=NS(num_prefill_module_buffer=in_phase if phase == "prefill" else other,
                                  num_decoding_module_buffer=other if phase == "prefill" else in_phase))

    class Wrapper(ExpertWrapperLike):                     # `phase` is a class attribute of Expert_Wrapper (Wrapper.py:434)
        pass

    Wrapper.phase = phase
    for e, ex in enumerate(blk.experts):
        wr = Wrapper(ex, L, e, eng, scales[e], cfg)
        wr.get_weights = e not in resident
        wrapped.append(wr)
    blk.experts = torch.nn.ModuleList(wrapped)
    if has_shared:
        blk.shared_experts = Wrapper(blk.shared_experts, L, -1, eng, sscale, cfg)
    for rep in range(2):                                  # the second call starts from a pool in mid-cycle
        out = first(blk(x))
        torch.cuda.synchronize()
        assert torch.equal(out, ref), rep
    check_against_oracle(resident_blk, w, x_cpu, out, blk)
    assert eng.max_held <= max(n_slots, 1) and not eng.held
    gets = [c[1] for c in eng.calls if c[0] == "get"]
    frees = [c[1] for c in eng.calls if c[0] == "free"]
    assert sorted(gets) == sorted(frees) == sorted(list(weights) * 2)
    assert not any(f"routed_expert_{L}_{e}" in gets for e in resident)
    assert ("clear", L, 0) in eng.calls


@pytest.mark.parametrize("routed_slots", [16, 5])
def test_block_with_library_stager(routed_slots):
    """Same, with the library's own Stager delivering fp8 experts from pinned host memory, with a
    pool as large as the layer and with one smaller than it (waves)."""
    from moe_gen_amd import StagedExpert, Stager, synthetic
    w = synthetic.WORKLOADS["deepseek_v3_w8a16"].scaled(n=256, h=512, I=256, E=16, n_group=4, topk_group=2, k=4, seq=64)
    blk = synthetic.build_block(w, device="cuda", gen_device="cpu")
    resident = synthetic.build_block(w, device="cuda", gen_device="cpu")
    x_cpu = synthetic.hidden_states(w, "cpu")
    x = x_cpu.cuda()
    blk.join_shared = False            # (as the staged walk runs it: the shared expert in a call of its own)
    ref = blk(x).clone()
    names = blk.experts[0].names
    fp8 = torch.float8_e4m3fn
    shapes = {"routed_expert": {f"{n}.weight": (tuple(getattr(blk.experts[0], n).weight.shape), fp8) for n in names},
              "shared_expert": {f"{n}.weight": (tuple(getattr(blk.shared_experts, n).weight.shape), fp8) for n in names}}
    st = Stager(shapes, {"routed_expert": routed_slots, "shared_expert": 1}, model_type="deepseek_v3", num_hidden_layers=8,
                num_local_experts=w.E)
    L = 5
    wrapped = []
    for e, ex in enumerate(blk.experts):
        st.add_module(f"routed_expert_{L}_{e}", "routed_expert",
                      {f"{n}.weight": getattr(ex, n).weight.data.cpu().pin_memory() for n in names})
        scales = {f"{n}.weight_scale_inv": getattr(ex, n).weight_scale_inv.data for n in names}
        for n in names:                                    # the resident copy is gone: a stale pointer would show
            getattr(ex, n).weight.data = torch.zeros(1, dtype=fp8, device="cuda")
        wrapped.append(StagedExpert(ex, L, e, st, scales))
    sh = blk.shared_experts
    st.add_module(f"shared_expert_{L}", "shared_expert", {f"{n}.weight": getattr(sh, n).weight.data.cpu().pin_memory() for n in names})
    blk.experts = torch.nn.ModuleList(wrapped)
    blk.shared_experts = StagedExpert(sh, L, -1, st, {f"{n}.weight_scale_inv": getattr(sh, n).weight_scale_inv.data for n in names})
    for _ in range(3):                                    # slots are recycled between calls
        out = blk(x)
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
    check_against_oracle(resident, w, x_cpu, out, blk)
    assert st.stats()[0] >= 3 * (w.E + 1)
    st.close()


@pytest.mark.parametrize("routed_slots", [64, 6])
def test_block_with_routing_aware_staging(routed_slots):
    """With per-expert token counts on the host, only experts that received tokens are staged
    (busiest first when they fit the pool, else in waves); the output is bit-identical to resident
    weights, in parity with the oracle, and the copy count equals the number of such experts.  The
    reference's worker copies every expert of the layer."""
    from moe_gen_amd import StagedExpert, Stager, synthetic
    w = synthetic.WORKLOADS["deepseek_v3_w8a16"].scaled(n=24, h=512, I=256, E=64, n_group=8, topk_group=4, k=4, seq=8)
    blk = synthetic.build_block(w, device="cuda", gen_device="cpu")
    resident = synthetic.build_block(w, device="cuda", gen_device="cpu")
    x_cpu = synthetic.hidden_states(w, "cpu")
    x = x_cpu.cuda()
    blk.join_shared = False            # (as the staged walk runs it: the shared expert in a call of its own)
    ref = blk(x).clone()
    used = int((blk.last_counts > 0).sum())
    assert routed_slots < used < w.E or routed_slots == w.E    # 24 tokens x 4 slots cannot reach all 64 experts
    names = blk.experts[0].names
    fp8 = torch.float8_e4m3fn
    shapes = {"routed_expert": {f"{n}.weight": (tuple(getattr(blk.experts[0], n).weight.shape), fp8) for n in names},
              "shared_expert": {f"{n}.weight": (tuple(getattr(blk.shared_experts, n).weight.shape), fp8) for n in names}}
    st = Stager(shapes, {"routed_expert": routed_slots, "shared_expert": 1}, model_type="deepseek_v3", num_hidden_layers=8,
                num_local_experts=w.E)
    st.set_policy("routed_expert", "on_demand")
    L = 5
    wrapped = []
    for e, ex in enumerate(blk.experts):
        st.add_module(f"routed_expert_{L}_{e}", "routed_expert",
                      {f"{n}.weight": getattr(ex, n).weight.data.cpu().pin_memory() for n in names})
        scales = {f"{n}.weight_scale_inv": getattr(ex, n).weight_scale_inv.data for n in names}
        for n in names:                                    # the resident copy is gone: a stale pointer would show
            getattr(ex, n).weight.data = torch.zeros(1, dtype=fp8, device="cuda")
        wrapped.append(StagedExpert(ex, L, e, st, scales))
    sh = blk.shared_experts
    st.add_module(f"shared_expert_{L}", "shared_expert", {f"{n}.weight": getattr(sh, n).weight.data.cpu().pin_memory() for n in names})
    blk.experts = torch.nn.ModuleList(wrapped)
    blk.shared_experts = StagedExpert(sh, L, -1, st, {f"{n}.weight_scale_inv": getattr(sh, n).weight_scale_inv.data for n in names})
    blk.routing_aware_staging = True
    assert st.pump() == 1                                  # the shared expert (cyclic) is prefetched; no routed expert
    for rep in range(3):
        c0 = st.stats()[0]
        out = blk(x)
        torch.cuda.synchronize()
        assert torch.equal(out, ref), rep
        assert st.stats()[0] - c0 == used + 1, (rep, st.stats()[0] - c0, used)   # + the shared expert
        assert not any(st.resident(f"routed_expert_{L}_{e}") for e in range(w.E))
    check_against_oracle(resident, w, x_cpu, out, blk)
    st.close()


def test_arena_to_hbm():
    """Modules registered from a pinned arena through its wire-format index arrive byte for byte."""
    from moe_gen_amd import Arena, Stager
    shapes = {"routed_expert": {"gate_proj.weight": ((64, 128), torch.float8_e4m3fn),
                                "up_proj.weight": ((64, 128), torch.float8_e4m3fn),
                                "down_proj.weight": ((128, 64), torch.float8_e4m3fn)}}
    g = torch.Generator().manual_seed(1)
    mods = {f"routed_expert_2_{e}": {n: torch.randint(0, 255, s, generator=g, dtype=torch.uint8).view(d)
                                     for n, (s, d) in shapes["routed_expert"].items()} for e in range(6)}
    packed = Arena.pack(mods)
    arena = Arena.from_bytes(packed.index.serialize(), packed.data)       # what a second process would do
    assert arena.data.is_pinned()
    st = Stager(shapes, {"routed_expert": 3}, model_type="deepseek_v3", num_hidden_layers=4, num_local_experts=6)
    for mk in mods:
        st.add_module_from_arena(mk, "routed_expert", arena)
    for rep in range(2):
        for mk, tensors in mods.items():
            w = st.get_weights(mk)
            torch.cuda.synchronize()
            for n, t in tensors.items():
                assert torch.equal(w[n].view(torch.uint8).cpu(), t.view(torch.uint8)), (mk, n)
            st.free_weights_buffer(mk)
    st.close()


@pytest.mark.parametrize("chunk_bytes", [1 << 16, 1 << 22])
def test_segment_to_hbm_through_the_bounce_ring(chunk_bytes):
    """Modules registered from a weight segment in ORDINARY host memory (Arena.stream_from: nothing is copied into
    pinned memory up front) arrive in their HBM slots byte for byte through the stager's ring of pinned chunks --
    pieces smaller than a chunk and pieces of many chunks, more modules than slots, three passes -- while the
    consumer's stream only ever waits on events."""
    from moe_gen_amd import Arena, Stager
    shapes = {"routed_expert": {"gate_proj.weight": ((256, 1024), torch.float8_e4m3fn),      # 256 KiB
                                "up_proj.weight": ((256, 1024), torch.float8_e4m3fn),
                                "down_proj.weight": ((1024, 2560), torch.float8_e4m3fn),     # 2.5 MiB
                                "tiny": ((3, 5), torch.float32)}}
    print(f"bounce ring, chunks of {chunk_bytes} bytes", flush=True)
    g = torch.Generator().manual_seed(2)
    mods = {f"routed_expert_{L}_{e}": {n: (torch.randint(0, 255, s, generator=g, dtype=torch.uint8).view(d) if d != torch.float32
                                           else torch.randn(s, generator=g))
                                       for n, (s, d) in shapes["routed_expert"].items()} for L in (2, 3, 4) for e in range(6)}
    packed = Arena.pack(mods, pin=False)
    arena = Arena.stream_from(packed.index.serialize(), packed.data)
    assert arena.pageable and not arena.data.is_pinned()
    st = Stager(shapes, {"routed_expert": 4}, model_type="deepseek_v3", num_hidden_layers=5, num_local_experts=6,
                bounce_chunks=4, bounce_chunk_bytes=chunk_bytes, bounce_threads=4)
    for mk in mods:
        st.add_module_from_arena(mk, "routed_expert", arena)
    for rep in range(3):
        for mk, tensors in mods.items():
            w = st.get_weights(mk)
            got = {n: t.clone() for n, t in w.items()}          # on the current stream, behind the hand-off event
            st.free_weights_buffer(mk)
            torch.cuda.synchronize()
            for n, t in tensors.items():
                assert torch.equal(got[n].view(torch.uint8).cpu(), t.view(torch.uint8)), (rep, mk, n)
    copies, nbytes = st.stats()
    assert copies >= 3 * len(mods)
    st.close()


@pytest.mark.parametrize("n", [0, 1, 60, 255, 256, 257, 1536])
def test_write_words_carries_a_pointer_table_in_kernel_arguments(n):
    """moe_write_words: the words arrive bit for bit, in order, and nothing next to them is touched; the host
    array may be overwritten as soon as the call has returned (the values travelled with the launch)."""
    import ctypes

    import numpy as np
    from moe_gen_amd import _native as N

    rng = np.random.default_rng(n)
    vals = rng.integers(0, 2**63, size=n, dtype=np.uint64) | (rng.integers(0, 2, size=n, dtype=np.uint64) << np.uint64(63))
    dev = torch.full((n + 2,), -7, dtype=torch.int64, device="cuda")
    arr = (ctypes.c_uint64 * max(n, 1))(*[int(v) for v in vals])
    st = torch.cuda.current_stream().cuda_stream
    N.check(N.lib().moe_write_words(dev.data_ptr() + 8, arr, n, st), "moe_write_words")
    for i in range(n):
        arr[i] = 0
    got = dev.cpu().numpy().view(np.uint64)
    assert got[0] == np.uint64(2**64 - 7) and got[-1] == np.uint64(2**64 - 7)
    assert (got[1:-1] == vals).all()
    assert N.lib().moe_write_words(dev.data_ptr() + 4, arr, 1, st) != 0      # misaligned destination is refused


def test_releases_of_a_wave_share_one_event_and_refill_when_nothing_is_held():
    """Releases only note the consumer's stream; the refills start with the release that leaves nothing held (or
    with the next call that copies), behind ONE event for the whole batch -- and the slots then hold the right
    modules' bytes however often the pool has gone round."""
    from moe_gen_amd import Stager
    shapes = {"routed_expert": {"w": ((256, 256), torch.bfloat16)}}
    st = Stager(shapes, {"routed_expert": 4}, model_type="mixtral", num_hidden_layers=4, num_local_experts=12)
    host = {}
    for e in range(12):
        host[e] = torch.randn(256, 256).to(torch.bfloat16).pin_memory()
        st.add_module(f"routed_expert_0_{e}", "routed_expert", {"w": host[e]})
    st.pump()
    assert st.stats()[0] == 4                                   # the pool is full: modules 0-3
    a = st.get_weights("routed_expert_0_0")["w"]
    b = st.get_weights("routed_expert_0_1")["w"]
    assert torch.equal(a.cpu(), host[0]) and torch.equal(b.cpu(), host[1])
    st.free_weights_buffer("routed_expert_0_0")
    assert st.stats()[0] == 4                                   # module 1 is still held: no refill yet
    st.free_weights_buffer("routed_expert_0_1")
    assert st.stats()[0] == 6                                   # nothing held: both freed slots are refilled (4, 5)
    # a held module does not stop an explicit pump, or the acquire of a module that needs a slot
    c = st.get_weights("routed_expert_0_2")["w"]
    d = st.get_weights("routed_expert_0_3")["w"]
    st.free_weights_buffer("routed_expert_0_2")
    assert st.stats()[0] == 6
    assert st.pump() == 1 and st.stats()[0] == 7                # module 6 into the slot of module 2
    assert torch.equal(d.cpu(), host[3])
    st.free_weights_buffer("routed_expert_0_3")
    # several trips round the pool, two modules at a time, with work on the stream between acquire and release
    x = torch.zeros(256, 256, device="cuda")
    order = [4, 5, 6, 7, 8, 9, 10, 11, 0, 1, 2, 3, 4, 5, 6, 7]
    for i in range(0, len(order), 2):
        pair = order[i:i + 2]
        got = [st.get_weights(f"routed_expert_0_{e}")["w"] for e in pair]
        for e, w in zip(pair, got):
            x += w.float() @ w.float().t()                       # keeps the slots busy on the stream
            assert torch.equal(w.cpu(), host[e]), e
        for e in pair:
            st.free_weights_buffer(f"routed_expert_0_{e}")
    st.sync()
    st.close()
