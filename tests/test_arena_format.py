"""Weight-arena index: the C implementation against the Python restatement of the reference's wire
format and against a byte string written out by hand from the format definition
(posix_shm.cpp:167-357); the arena feeding the stager (host backend)."""
import random

import pytest
import torch

from moe_gen_amd import Arena, ArenaIndex, Stager
from oracle import arena_format as F

# {"a": {"w": tensor_meta(offset=16, byte_size=8, shape=[2, 2])}}, written out field by field
HAND = bytes.fromhex(
    "0100000000000000"          # 1 module
    "0100000000000000" "61"     # key length 1, "a"
    "0100000000000000"          # 1 tensor
    "0100000000000000" "77"     # key length 1, "w"
    "1000000000000000"          # offset 16
    "0800000000000000"          # byte_size 8
    "0200000000000000"          # 2 dims
    "0200000000000000" "0200000000000000")


def random_map(rng, n_modules=5):
    m = {}
    for i in range(n_modules):
        inner = {}
        for j in range(rng.randint(0, 4)):
            shape = tuple(rng.randint(1, 9000) for _ in range(rng.randint(0, 4)))
            inner[f"proj{j}.weight" + "x" * rng.randint(0, 3)] = (rng.randint(0, 2 ** 40), rng.randint(0, 2 ** 33), shape)
        m[f"routed_expert_{rng.randint(0, 60)}_{i}"] = inner
    return m


def build(m):
    ix = ArenaIndex()
    for mk, inner in m.items():
        for tk, (off, nb, shape) in inner.items():
            ix.add(mk, tk, off, nb, shape)
    return ix


def test_hand_written_vector():
    assert F.serialize({"a": {"w": (16, 8, (2, 2))}}) == HAND and F.serialized_size({"a": {"w": (16, 8, (2, 2))}}) == len(HAND)
    assert F.deserialize(HAND) == {"a": {"w": (16, 8, (2, 2))}}
    ix = ArenaIndex.parse(HAND)
    assert ix.modules() == {"a": {"w": (16, 8, (2, 2))}}
    assert ix.serialize() == HAND
    assert build({"a": {"w": (16, 8, (2, 2))}}).serialize() == HAND


def test_round_trip_and_cross_parse():
    rng = random.Random(7)
    for trial in range(20):
        m = {k: v for k, v in random_map(rng).items() if v}      # a module exists once it has a tensor
        wire = build(m).serialize()
        assert wire == F.serialize(m) and len(wire) == F.serialized_size(m)
        assert ArenaIndex.parse(F.serialize(m)).modules() == m
        assert F.deserialize(wire) == m
    empty = ArenaIndex()
    assert empty.serialize() == F.serialize({}) == b"\0" * 8 and ArenaIndex.parse(b"\0" * 8).modules() == {}
    # a module with no tensors survives the wire (the reference writes inner size 0)
    wire = F.serialize({"shared_expert_3": {}, "b": {"t": (0, 4, ())}})
    assert ArenaIndex.parse(wire).modules() == {"shared_expert_3": {}, "b": {"t": (0, 4, ())}}
    assert ArenaIndex.parse(wire).serialize() == wire
    # a repeated key overwrites, as assignment into the reference's map does
    ix = build({"m": {"t": (0, 4, (1,))}})
    ix.add("m", "t", 64, 8, (2,))
    assert ix.modules() == {"m": {"t": (64, 8, (2,))}}
    assert "m" in ix and "n" not in ix


def test_truncated_buffers_fail_like_the_reference():
    m = {"routed_expert_3_0": {"gate_proj.weight": (0, 64, (4, 8)), "up_proj.weight": (256, 64, (4, 8))}}
    wire = F.serialize(m)
    for cut in range(len(wire)):
        with pytest.raises(RuntimeError, match="Buffer overflow") as e_c:
            ArenaIndex.parse(wire[:cut])
        with pytest.raises(RuntimeError, match="Buffer overflow") as e_py:
            F.deserialize(wire[:cut])
        # same field named by both
        assert str(e_py.value) in str(e_c.value), (cut, str(e_c.value), str(e_py.value))
    # an absurd dimension count must not allocate
    bad = bytearray(wire)
    pos = wire.index(b"gate_proj.weight") + len(b"gate_proj.weight") + 16
    bad[pos:pos + 8] = (2 ** 62).to_bytes(8, "little")
    with pytest.raises(RuntimeError, match="tensor_shape data"):
        ArenaIndex.parse(bytes(bad))
    with pytest.raises(RuntimeError, match="negative"):
        ArenaIndex().add("m", "t", -1, 4, (1,))


SHAPES = {"routed_expert": {"gate_proj.weight": ((4, 8), torch.bfloat16), "up_proj.weight": ((4, 8), torch.bfloat16),
                            "down_proj.weight": ((8, 4), torch.bfloat16)}}


def test_arena_feeds_the_stager():
    g = torch.Generator().manual_seed(0)
    mods = {f"routed_expert_0_{e}": {n: torch.randn(s, generator=g).to(d) for n, (s, d) in SHAPES["routed_expert"].items()}
            for e in range(5)}
    packed = Arena.pack(mods, pin=False)
    # the arena travels as (index bytes, data bytes), e.g. between processes
    arena = Arena.from_bytes(packed.index.serialize(), packed.data.numpy().tobytes(), pin=False)
    assert arena.index.modules() == packed.index.modules()
    for mk, tensors in mods.items():
        for tk, t in tensors.items():
            assert torch.equal(arena.tensor(mk, tk, t.dtype), t)
    st = Stager(SHAPES, {"routed_expert": 2}, backend="host", model_type="mixtral", num_hidden_layers=1, num_local_experts=5)
    for mk in mods:
        st.add_module_from_arena(mk, "routed_expert", arena)
    for mk, tensors in mods.items():
        w = st.get_weights(mk)
        assert all(torch.equal(w[n], tensors[n]) for n in tensors), mk
        st.free_weights_buffer(mk)
    with pytest.raises(RuntimeError, match="Module key not found in storage"):
        st.add_module_from_arena("routed_expert_9_9", "routed_expert", arena)
    # an entry that points outside the data blob is refused when the module is registered
    ix = ArenaIndex.parse(packed.index.serialize())
    ix.add("routed_expert_0_0", "gate_proj.weight", packed.data.numel() - 8, 64, (4, 8))
    with pytest.raises(RuntimeError, match="outside"):
        st.add_module_from_arena("routed_expert_0_0", "routed_expert", Arena(ix, packed.data))
    # a shape that does not match the slot layout is refused
    ix2 = ArenaIndex.parse(packed.index.serialize())
    ix2.add("routed_expert_0_1", "gate_proj.weight", 0, 64, (8, 4))
    with pytest.raises(RuntimeError, match="does not match"):
        st.add_module_from_arena("routed_expert_0_1", "routed_expert", Arena(ix2, packed.data))
    st.close()


def test_golden_wire_fixture():
    """tests/golden/arena_index.bin against its JSON description: both parsers, and both writers
    reproduce the bytes."""
    import json
    import os
    here = os.path.join(os.path.dirname(__file__), "golden")
    wire = open(os.path.join(here, "arena_index.bin"), "rb").read()
    want = {mk: {tk: (o, nb, tuple(sh)) for tk, (o, nb, sh) in inner.items()}
            for mk, inner in json.load(open(os.path.join(here, "arena_index.json"))).items()}
    assert F.deserialize(wire) == want
    ix = ArenaIndex.parse(wire)
    assert ix.modules() == want and list(ix.modules()) == list(want)
    assert ix.serialize() == wire and build(want).serialize() == wire and F.serialize(want) == wire
