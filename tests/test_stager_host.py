"""The slot pool / copy queue of libmoe_mi355.so with its host-memcpy backend, against the
pure-Python model of the reference's GPU_Weight_Buffer + HtoD worker (oracle.SlotPoolModel)."""
import pytest
import torch

from moe_gen_amd import Stager
from oracle.oracle import SlotPoolModel

SHAPES = {"routed_expert": {"gate_proj.weight": ((4, 8), torch.bfloat16), "up_proj.weight": ((4, 8), torch.bfloat16),
                            "down_proj.weight": ((8, 4), torch.bfloat16)},
          "shared_expert": {"gate_proj.weight": ((8, 8), torch.bfloat16), "up_proj.weight": ((8, 8), torch.bfloat16),
                            "down_proj.weight": ((8, 8), torch.bfloat16)}}


def make(model_type, layers, E, slots, first_moe):
    st = Stager(SHAPES, {"routed_expert": slots, "shared_expert": 1}, backend="host", model_type=model_type,
                num_hidden_layers=layers, num_local_experts=E)
    names = {"routed_expert": [], "shared_expert": []}
    host = {}
    g = torch.Generator().manual_seed(0)
    for L in range(first_moe, layers):
        key = f"shared_expert_{L}"
        host[key] = {n: torch.randn(s, generator=g).to(d) for n, (s, d) in SHAPES["shared_expert"].items()}
        st.add_module(key, "shared_expert", host[key]); names["shared_expert"].append(key)
        for e in range(E):
            key = f"routed_expert_{L}_{e}"
            host[key] = {n: torch.randn(s, generator=g).to(d) for n, (s, d) in SHAPES["routed_expert"].items()}
            st.add_module(key, "routed_expert", host[key]); names["routed_expert"].append(key)
    model = SlotPoolModel({"routed_expert": slots, "shared_expert": 1}, names, model_type, layers, E)
    return st, model, host, names


def model_get(model, key):
    while key not in model.resident:
        assert model.pump(), f"model cannot schedule {key}"


@pytest.mark.parametrize("model_type,first_moe", [("deepseek_v2", 1), ("deepseek_v3", 3), ("mixtral", 0)])
def test_fifo_reuse_and_clear_rule(model_type, first_moe):
    layers, E, slots = first_moe + 3, 6, 4
    st, model, host, names = make(model_type, layers, E, slots, first_moe)
    st.pump()
    while model.pump():
        pass
    for rounds in range(2):                                  # two passes over the model: wrap-around
        for L in range(first_moe, layers):
            key = f"shared_expert_{L}"
            w = st.get_weights(key); model_get(model, key)
            assert all(torch.equal(w[n], host[key][n]) for n in w)
            st.free_weights_buffer(key); model.release(key)
            while model.pump():
                pass
            for e in range(E):
                if (e + L + rounds) % 3 == 0:
                    continue                                 # expert received no tokens: never fetched
                st.clear_expert_buffer(L, e); model.clear_expert_buffer(L, e)
                while model.pump():
                    pass
                key = f"routed_expert_{L}_{e}"
                w = st.get_weights(key); model_get(model, key)
                for n in w:                                   # byte-for-byte content after the copy
                    assert torch.equal(w[n], host[key][n]), (key, n)
                st.free_weights_buffer(key); model.release(key)
                while model.pump():
                    pass
                for k2 in names["routed_expert"]:
                    assert st.resident(k2) == (k2 in model.resident), (key, k2)
    copies, nbytes = st.stats()
    assert copies == len(model.copies)


@pytest.mark.parametrize("model_type,layers,wrapping", [("deepseek_v3", 6, (0, 1, 2, 3)), ("deepseek_v2", 27, (0, 1)),
                                                        ("mixtral", 4, ())])
def test_clear_rule_through_the_c_abi(model_type, layers, wrapping):
    """moe_stage_clear_expert_buffer, driven by module tags through ctypes alone: experts below
    expert_idx of the layer and every routed expert of the previous layer are released, the first
    layers of the DeepSeek models take the last layer as previous (GPU_Weight_Buffer.cpp:279-294),
    shared experts and other layers stay.  Checked against the Python slot-pool model."""
    import ctypes
    from moe_gen_amd import _native as N
    L = N.lib()
    E, nb = 3, 64
    probe = sorted({0, 1, 2, 3, 4, layers - 1})               # layers that hold modules
    n_mod = len(probe) * (E + 1)
    pool = (ctypes.c_uint8 * (n_mod * nb))()
    spool = (ctypes.c_uint8 * (len(probe) * nb))()
    h = ctypes.c_void_p()
    N.check(L.moe_stage_create(ctypes.byref(h), 2, (ctypes.c_size_t * 2)(nb, nb), (ctypes.c_int32 * 2)(len(probe) * E, len(probe)),
                               (ctypes.c_void_p * 2)(ctypes.addressof(pool), ctypes.addressof(spool)), 1), "create")
    N.check(L.moe_stage_set_model(h, model_type.encode(), layers, E), "set_model")
    src = (ctypes.c_uint8 * nb)(*range(nb))
    ids, names = {}, {"routed_expert": [], "shared_expert": []}
    for lay in probe:
        for e in list(range(E)) + [-1]:
            mid = L.moe_stage_add_module(h, 0 if e >= 0 else 1, 1, (ctypes.c_void_p * 1)(ctypes.addressof(src)),
                                         (ctypes.c_size_t * 1)(nb), (ctypes.c_size_t * 1)(0))
            assert mid >= 0
            N.check(L.moe_stage_tag_module(h, mid, lay, e), "tag")
            key = f"routed_expert_{lay}_{e}" if e >= 0 else f"shared_expert_{lay}"
            ids[key] = mid
            names["routed_expert" if e >= 0 else "shared_expert"].append(key)
    for lay in probe:
        for upto in (0, 2):
            # every module fits the pool: all resident before each clear, in the library and in a fresh model
            model = SlotPoolModel({"routed_expert": len(probe) * E, "shared_expert": len(probe)}, names, model_type, layers, E)
            for _ in range(n_mod):
                model.pump()
            assert L.moe_stage_pump(h) >= 0
            assert all(L.moe_stage_resident(h, i) == 1 for i in ids.values()) and len(model.resident) == n_mod
            before = set(model.resident)
            model.clear_expert_buffer(lay, upto)
            released = L.moe_stage_clear_expert_buffer(h, lay, upto, None)
            assert released == len(before - set(model.resident))
            prev = layers - 1 if lay in wrapping else lay - 1
            want_gone = {f"routed_expert_{lay}_{e}" for e in range(upto)} | {f"routed_expert_{prev}_{e}" for e in range(E)}
            assert before - set(model.resident) == want_gone & set(ids)
            # the freed slots are refilled at once with the modules that are not resident
            assert all(L.moe_stage_resident(h, i) == 1 for i in ids.values())
    assert L.moe_stage_tag_module(h, 10 ** 6, 0, 0) == -1 and "unknown module" in N.last_error()
    L.moe_stage_destroy(h)


def test_release_out_of_order_does_not_block_the_queue():
    """Five modules, four slots, the consumer lets go of a later module first: the freed slot takes
    the next module in line that is not resident, and a later acquire of the released module finds
    a slot.  (The reference's worker would copy the still-resident head a second time.)"""
    st = Stager(SHAPES, {"routed_expert": 4, "shared_expert": 1}, backend="host", model_type="mixtral",
                num_hidden_layers=1, num_local_experts=5)
    for e in range(5):
        st.add_module(f"routed_expert_0_{e}", "routed_expert",
                      {n: torch.full(s, float(e)).to(d) for n, (s, d) in SHAPES["routed_expert"].items()})
    for e in range(4):
        st.get_weights(f"routed_expert_0_{e}")
    st.free_weights_buffer("routed_expert_0_1")                # 4 takes the slot; queue head 0 is still held
    assert st.resident("routed_expert_0_4") and not st.resident("routed_expert_0_1")
    st.free_weights_buffer("routed_expert_0_2")                # heads 0 (held) and 4 (resident) keep their place: 1 is copied
    assert st.resident("routed_expert_0_1")
    w = st.get_weights("routed_expert_0_1")
    assert float(w["gate_proj.weight"][0, 0]) == 1.0
    assert st.stats()[0] == 6


def test_reset_is_refused_while_a_module_is_held():
    st = Stager(SHAPES, {"routed_expert": 2, "shared_expert": 1}, backend="host", model_type="mixtral",
                num_hidden_layers=1, num_local_experts=3)
    for e in range(3):
        st.add_module(f"routed_expert_0_{e}", "routed_expert",
                      {n: torch.full(s, float(e)).to(d) for n, (s, d) in SHAPES["routed_expert"].items()})
    st.get_weights("routed_expert_0_0")
    with pytest.raises(RuntimeError, match="still held"):
        st.reset_prefill_buffer()
    st.free_weights_buffer("routed_expert_0_0")
    st.reset_prefill_buffer()
    assert not any(st.resident(f"routed_expert_0_{e}") for e in range(3))


def test_errors_and_phase_switch():
    st, model, host, names = make("mixtral", 2, 4, 2, 0)
    with pytest.raises(RuntimeError, match="Module key not found"):
        st.get_weights("routed_expert_7_7")
    st.get_weights("routed_expert_0_0"); st.get_weights("routed_expert_0_1")
    with pytest.raises(RuntimeError, match="every slot"):
        st.get_weights("routed_expert_0_2")                  # both slots held: the reference would spin forever
    with pytest.raises(RuntimeError, match="not resident"):
        st.free_weights_buffer("routed_expert_1_3")
    st.free_weights_buffer("routed_expert_0_0"); st.free_weights_buffer("routed_expert_0_1")
    # decoding phase may use more slots; back in prefill the engine resets residency and rewinds the
    # queue (moe_gen/engine.py:680-683)
    big = Stager(SHAPES, {"routed_expert": 2, "shared_expert": 1}, n_slots_decoding={"routed_expert": 5, "shared_expert": 1},
                 backend="host", model_type="mixtral", num_hidden_layers=1, num_local_experts=6)
    for e in range(6):
        big.add_module(f"routed_expert_0_{e}", "routed_expert",
                       {n: torch.full(s, float(e)).to(d) for n, (s, d) in SHAPES["routed_expert"].items()})
    assert big.pump() == 2
    big.set_phase("decoding")
    assert big.pump() == 3 and big.resident("routed_expert_0_4") and not big.resident("routed_expert_0_5")
    assert big.pool_size("routed_expert") == 5
    big.set_phase("prefill")
    assert big.resident("routed_expert_0_0")               # set_phase("prefill") alone changes nothing
    big.reset_prefill_buffer(); big.reset_weight_copy_queue()
    assert not big.resident("routed_expert_0_0") and big.pool_size("routed_expert") == 2
    with pytest.raises(RuntimeError, match="unknown phase"):
        big.set_phase("warmup")
    assert big.pump() == 2 and big.resident("routed_expert_0_1") and not big.resident("routed_expert_0_2")
    with pytest.raises(RuntimeError):
        big.add_module("routed_expert_0_9", "routed_expert", {"gate_proj.weight": torch.zeros(1)})


def test_on_demand_fetches_only_what_is_named():
    """Routing-aware staging: with the on-demand policy nothing is copied until named; fetch()
    copies the named modules in the given order into the first free slots, skips resident ones,
    and fails when the pool is full.  Checked against the Python slot-pool model and by content."""
    layers, E, slots = 2, 8, 5
    st, model, host, names = make("mixtral", layers, E, slots, 0)
    st.set_policy("routed_expert", "on_demand"); model.on_demand.add("routed_expert")
    assert st.pump() == 1                                  # only the (cyclic) shared expert moves
    while model.pump():
        pass
    assert not any(st.resident(k) for k in names["routed_expert"])
    rng = torch.Generator().manual_seed(3)
    for step in range(12):
        L = step % layers
        counts = torch.randint(0, 4, (E,), generator=rng) * (torch.rand(E, generator=rng) < 0.6)
        hot = sorted((e for e in range(E) if counts[e] > 0), key=lambda e: -int(counts[e]))[:slots]
        keys = [f"routed_expert_{L}_{e}" for e in hot]
        assert st.fetch(keys) == model.fetch(keys) == len(keys)
        assert st.fetch(keys) == 0                         # already resident: nothing to do
        for k2 in names["routed_expert"]:
            assert st.resident(k2) == (k2 in model.resident), (step, k2)
        for key in keys:
            w = st.get_weights(key)
            assert all(torch.equal(w[n], host[key][n]) for n in w), key
        for key in keys:
            st.free_weights_buffer(key); model.release(key)
        assert not any(st.resident(k) for k in names["routed_expert"])   # a freed slot is not refilled
    assert st.stats()[0] == len(model.copies)
    # get_weights on a module nobody fetched stages it alone
    w = st.get_weights("routed_expert_1_7")
    assert all(torch.equal(w[n], host["routed_expert_1_7"][n]) for n in w)
    # pool exhausted: 4 more fit, the 5th does not
    assert st.fetch([f"routed_expert_0_{e}" for e in range(4)]) == 4
    with pytest.raises(RuntimeError, match="no free slot"):
        st.fetch(["routed_expert_0_4", "routed_expert_0_5"])
    with pytest.raises(RuntimeError, match="Module key not found"):
        st.fetch(["routed_expert_9_9"])
    with pytest.raises(RuntimeError, match="unknown staging policy"):
        st.set_policy("routed_expert", "sometimes")
    # back to the reference's policy: the queue resumes where it stood
    for e in range(4):
        st.free_weights_buffer(f"routed_expert_0_{e}")
    st.free_weights_buffer("routed_expert_1_7")
    st.set_policy("routed_expert", "cyclic")
    assert st.pump() == slots and st.resident("routed_expert_0_0")


def test_fetch_takes_over_slots_nobody_asked_for():
    """Slots filled by the cyclic prefetch before a type was switched to on-demand hold modules that
    no consumer acquired and no fetch named: a fetch that finds no free slot takes those over instead
    of failing, but never a held module or one an earlier fetch named."""
    E, slots = 6, 3
    st = Stager(SHAPES, {"routed_expert": slots, "shared_expert": 1}, backend="host", model_type="mixtral",
                num_hidden_layers=2, num_local_experts=E)
    host = {}
    for L in range(2):
        for e in range(E):
            key = f"routed_expert_{L}_{e}"
            host[key] = {n: torch.full(s, float(10 * L + e)).to(d) for n, (s, d) in SHAPES["routed_expert"].items()}
            st.add_module(key, "routed_expert", host[key])
    assert st.pump() == slots                               # cyclic: experts 0..2 of layer 0 fill the pool
    st.set_policy("routed_expert", "on_demand")
    assert st.fetch(["routed_expert_1_4", "routed_expert_1_5"]) == 2     # two of the three prefetched modules give way
    assert sum(st.resident(f"routed_expert_0_{e}") for e in range(3)) == 1
    w = st.get_weights("routed_expert_1_4")
    assert float(w["gate_proj.weight"][0, 0]) == 14.0
    assert st.fetch(["routed_expert_1_0"]) == 1             # the last prefetched module gives way
    assert not any(st.resident(f"routed_expert_0_{e}") for e in range(3))
    with pytest.raises(RuntimeError, match="no free slot"):  # held (1_4) and named (1_5, 1_0) modules stay
        st.fetch(["routed_expert_1_1"])
    st.free_weights_buffer("routed_expert_1_4")
    assert st.fetch(["routed_expert_1_1"]) == 1
    for key in ("routed_expert_1_5", "routed_expert_1_0", "routed_expert_1_1"):
        w = st.get_weights(key)
        assert all(torch.equal(w[n], host[key][n]) for n in w)
        st.free_weights_buffer(key)


def test_pool_size_in_the_decoding_phase_follows_the_pool():
    """A type without a decoding entry keeps its prefill slots; a decoding count below the prefill
    count does not shrink the pool (the C side runs with the larger of the two)."""
    st = Stager(SHAPES, {"routed_expert": 4, "shared_expert": 2}, n_slots_decoding={"routed_expert": 3}, backend="host",
                model_type="mixtral", num_hidden_layers=1, num_local_experts=4)
    st.set_phase("decoding")
    assert st.pool_size("routed_expert") == 4 and st.pool_size("shared_expert") == 2
    st2 = Stager(SHAPES, {"routed_expert": 2, "shared_expert": 1}, n_slots_decoding={"routed_expert": 6}, backend="host",
                 model_type="mixtral", num_hidden_layers=1, num_local_experts=4)
    assert st2.pool_size("routed_expert") == 2
    st2.set_phase("decoding")
    assert st2.pool_size("routed_expert") == 6 and st2.pool_size("shared_expert") == 1


@pytest.mark.parametrize("chunk_bytes,threads", [(4096, 1), (8192, 3), (1 << 22, 4)])
def test_pageable_segment_through_the_bounce_ring(chunk_bytes, threads):
    """A weight segment adopted where it lies, in ordinary host memory (Arena.stream_from: the reference maps its
    shm segment once and views it, Weights_Storage.cpp:52-78), reaches the slots through the stager's ring of
    bounce chunks byte for byte: pieces smaller than, equal to and several times a chunk, more modules than slots,
    several passes (chunks and slots are reused), skipped modules reclaimed by clear_expert_buffer, and a reset in
    between.  Host backend: the chunks are plain memory and the transfer out of a chunk is a memcpy."""
    from moe_gen_amd import Arena
    shapes = {"routed_expert": {"gate_proj.weight": ((96, 128), torch.bfloat16),        # 24576 bytes
                                "up_proj.weight": ((32, 128), torch.bfloat16),          # 8192
                                "down_proj.weight": ((1300, 1024), torch.float32)}}     # 5.3 MB: above 1 MiB per thread
    E, L, slots = 5, 3, 3        # (three layers: with two, the layer before the current one is also the next one, and
    g = torch.Generator().manual_seed(5)   #  the rule that drops the previous layer's leftovers drops what was just prefetched)
    mods = {f"routed_expert_{lay}_{e}": {n: torch.randn(s, generator=g).to(d) for n, (s, d) in shapes["routed_expert"].items()}
            for lay in range(L) for e in range(E)}
    packed = Arena.pack(mods, pin=False)
    assert not packed.data.is_pinned()
    arena = Arena.stream_from(packed.index.serialize(), packed.data)        # what a process that maps the segment does
    assert arena.pageable and arena.data.data_ptr() == packed.data.data_ptr()   # adopted in place, not copied
    st = Stager(shapes, {"routed_expert": slots}, backend="host", model_type="mixtral", num_hidden_layers=L,
                num_local_experts=E, bounce_chunks=3, bounce_chunk_bytes=chunk_bytes, bounce_threads=threads)
    for mk in mods:
        st.add_module_from_arena(mk, "routed_expert", arena)
    for rounds in range(3):
        for lay in range(L):
            for e in range(E):
                st.clear_expert_buffer(lay, e)
                if (e + rounds) % 4 == 3:
                    continue                              # skipped: its slot is reclaimed by a later clear
                key = f"routed_expert_{lay}_{e}"
                w = st.get_weights(key)
                for n, t in mods[key].items():
                    assert torch.equal(w[n], t), (rounds, key, n)
                st.free_weights_buffer(key)
        if rounds == 1:
            st.reset_prefill_buffer(); st.reset_weight_copy_queue()      # drains the worker's queue first
    st.sync()
    copies, nbytes = st.stats()
    per_module = sum(t.numel() * t.element_size() for t in mods["routed_expert_0_0"].values())
    assert copies >= 3 * L * (E - 2) and nbytes == copies * per_module
    st.close()


def test_pageable_module_without_a_bounce_ring_is_an_error():
    """Through the C ABI alone: a module registered as pageable cannot be copied before moe_stage_set_bounce."""
    import ctypes
    from moe_gen_amd import _native as N
    L = N.lib()
    nb = 256
    pool = (ctypes.c_uint8 * (2 * nb))()
    h = ctypes.c_void_p()
    N.check(L.moe_stage_create(ctypes.byref(h), 1, (ctypes.c_size_t * 1)(nb), (ctypes.c_int32 * 1)(2),
                               (ctypes.c_void_p * 1)(ctypes.addressof(pool)), 1), "create")
    src = (ctypes.c_uint8 * nb)(*range(nb))
    mid = L.moe_stage_add_module_pageable(h, 0, 1, (ctypes.c_void_p * 1)(ctypes.addressof(src)), (ctypes.c_size_t * 1)(nb),
                                          (ctypes.c_size_t * 1)(0))
    assert mid == 0
    slot = ctypes.c_int32(-1)
    assert L.moe_stage_acquire(h, mid, None, ctypes.byref(slot)) != 0 and "bounce" in N.last_error()
    assert L.moe_stage_set_bounce(h, 1, 4096, 1) == -1 and "n_chunks" in N.last_error()
    N.check(L.moe_stage_set_bounce(h, 2, 4096, 2), "set_bounce")
    assert L.moe_stage_set_bounce(h, 2, 4096, 2) == -1 and "already" in N.last_error()
    N.check(L.moe_stage_acquire(h, mid, None, ctypes.byref(slot)), "acquire")
    assert bytes(pool[slot.value * nb:(slot.value + 1) * nb]) == bytes(src)
    L.moe_stage_destroy(h)
