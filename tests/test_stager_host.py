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


def test_prev_layer_wraps_for_first_moe_layers():
    st, model, host, names = make("deepseek_v3", 6, 4, 4, 3)
    assert st._prev_layer(3) == 5 and st._prev_layer(4) == 3 and model.prev_layer(3) == 5
    st2 = Stager(SHAPES, {"routed_expert": 2, "shared_expert": 1}, backend="host", model_type="deepseek_v2",
                 num_hidden_layers=27, num_local_experts=4)
    assert st2._prev_layer(1) == 26 and st2._prev_layer(0) == 26 and st2._prev_layer(2) == 1


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
    # decoding phase may use more slots; prefill resets residency and rewinds the queue
    big = Stager(SHAPES, {"routed_expert": 2, "shared_expert": 1}, n_slots_decoding={"routed_expert": 5, "shared_expert": 1},
                 backend="host", model_type="mixtral", num_hidden_layers=1, num_local_experts=6)
    for e in range(6):
        big.add_module(f"routed_expert_0_{e}", "routed_expert",
                       {n: torch.full(s, float(e)).to(d) for n, (s, d) in SHAPES["routed_expert"].items()})
    assert big.pump() == 2
    big.set_phase("decoding")
    assert big.pump() == 3 and big.resident("routed_expert_0_4") and not big.resident("routed_expert_0_5")
    big.set_phase("prefill")
    assert not big.resident("routed_expert_0_0")
    assert big.pump() == 2 and big.resident("routed_expert_0_1") and not big.resident("routed_expert_0_2")
    with pytest.raises(RuntimeError):
        big.add_module("routed_expert_0_9", "routed_expert", {"gate_proj.weight": torch.zeros(1)})
