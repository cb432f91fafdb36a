"""Host-side behaviour of the blocks that needs no GPU: parameter tree, errors, no CPU fallback."""
import pytest
import torch

import moe_gen_amd as M
from moe_gen_amd import deepseek_v2, synthetic


def tiny(family):
    w = {"v3": synthetic.WORKLOADS["deepseek_v3_w8a16"], "v2": synthetic.WORKLOADS["deepseek_v2_236b"],
         "mixtral": synthetic.WORKLOADS["mixtral_8x7b"]}[family]
    return w.scaled(n=16, h=128, I=128, E=8 if family != "v2" else 16, seq=4,
                    n_group=4 if family != "mixtral" else 1, topk_group=2 if family != "mixtral" else 1,
                    k=2)


def test_parameter_tree_matches_the_reference_names():
    """Keys the reference's initializers address (deepseekv3_initializer.py:1109-1152,
    Mixtral_Initializer.py:691-716)."""
    b3 = synthetic.build_block(tiny("v3"), device="cpu")
    keys = set(dict(b3.named_parameters()))
    for k in ("gate.weight", "gate.e_score_correction_bias", "experts.0.gate_proj.weight", "experts.7.down_proj.weight",
              "experts.3.up_proj.weight", "shared_experts.gate_proj.weight", "experts.0.gate_proj.weight_scale_inv"):
        assert k in keys, k
    assert b3.experts[0].gate_proj.weight.dtype == torch.float8_e4m3fn
    b2 = synthetic.build_block(tiny("v2"), device="cpu")
    assert {"gate.weight", "experts.15.up_proj.weight", "shared_experts.down_proj.weight"} <= set(dict(b2.named_parameters()))
    assert not hasattr(b2.gate, "e_score_correction_bias")
    assert b2.shared_experts.gate_proj.weight.shape == (2 * 128, 128)        # intermediate = S * I
    bm = synthetic.build_block(tiny("mixtral"), device="cpu")
    assert {"gate.weight", "experts.0.w1.weight", "experts.0.w2.weight", "experts.7.w3.weight"} <= set(dict(bm.named_parameters()))
    assert bm.experts[0].w1.weight.shape == (128, 128) and bm.gate.weight.shape == (8, 128)


def test_no_cpu_fallback():
    for fam in ("v3", "v2", "mixtral"):
        w = tiny(fam)
        blk = synthetic.build_block(w, device="cpu")
        with pytest.raises(RuntimeError, match="GPU"):
            blk(synthetic.hidden_states(w, "cpu"))
    with pytest.raises((RuntimeError, TypeError)):
        M.ops.router(torch.zeros(4, 16, dtype=torch.bfloat16), torch.zeros(8, 16, dtype=torch.bfloat16), None,
                     M.ops.RouterSpec(8, 2))


def test_unsupported_rules_raise_like_the_reference():
    cfg = M.DeepseekV3Config(hidden_size=64, n_routed_experts=8, n_group=2, topk_group=1, num_experts_per_tok=2,
                             moe_intermediate_size=64, scoring_func="softmax")
    blk = M.DeepseekV3MoE(cfg).eval()
    with pytest.raises(NotImplementedError, match="insupportable scoring function"):
        blk(torch.zeros(1, 2, 64, dtype=torch.bfloat16))
    cfg2 = M.DeepseekV2Config(hidden_size=64, n_routed_experts=8, num_experts_per_tok=2, moe_intermediate_size=64,
                              topk_method="gready")          # the reference config's own default (a typo upstream)
    gate = deepseek_v2.MoEGate(cfg2).eval()
    with pytest.raises(NotImplementedError, match="insupportable TopK function"):
        gate(torch.zeros(1, 2, 64, dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError):
        M.DeepseekV3MoE(M.DeepseekV3Config(hidden_size=64, n_routed_experts=8, ep_size=2, moe_intermediate_size=64))
    with pytest.raises(NotImplementedError):
        M.DeepseekV3MLP(M.DeepseekV3Config(hidden_size=64, intermediate_size=64, hidden_act="gelu"))


def test_workload_table_matches_the_benchmark_definition():
    W = synthetic.WORKLOADS
    v3 = W["deepseek_v3_w8a16"]
    assert (v3.n, v3.h, v3.E, v3.k, v3.I, v3.S, v3.n_group, v3.topk_group, v3.scale, v3.fp8) == \
        (65536, 7168, 256, 8, 2048, 1, 8, 4, 2.5, True)
    assert abs(v3.routed_flop - 46179.5e9) / 46179.5e9 < 1e-4 and abs(v3.shared_flop - 5772.4e9) / 5772.4e9 < 1e-4
    assert abs(v3.dispatch_bytes / 2 ** 20 - 14338) < 1 and abs(v3.combine_bytes / 2 ** 20 - 8962) < 1
    assert abs(v3.router_bytes / 2 ** 20 - 903.5) < 0.1
    v2 = W["deepseek_v2_236b"]
    assert (v2.n, v2.h, v2.E, v2.k, v2.I, v2.S, v2.method, v2.scale) == (32768, 5120, 160, 6, 1536, 2,
                                                                        "group_limited_greedy", 16.0)
    assert abs(W["mixtral_8x7b"].routed_flop - 11544.9e9) / 11544.9e9 < 1e-4
    assert W["mixtral_8x22b_decode"].n == 256 and W["deepseek_v2_lite"].zipf == 1.1


def test_zipf_bias_rides_on_feature_zero():
    w = synthetic.WORKLOADS["deepseek_v2_lite"].scaled(n=64, h=64)
    x = synthetic.hidden_states(w)
    g = synthetic.gate_weight(w)
    assert (x.reshape(-1, 64)[:, 0] == 1).all()
    b = g[:, 0].float()
    assert abs(b.mean().item()) < 0.02 and b.max() > 2.0 and b.min() < -0.5   # centred log-Zipf, skewed
    assert torch.equal(g, synthetic.gate_weight(w))                           # deterministic in the seed


class _SlotLimitedEngine:
    """A stand-in for MoE-Gen's core_engine whose pool has `n_slots` slots and whose copy worker
    delivers modules in registration order (HtoD_Engine.cpp:201-268): get_weights of a module that
    is not deliverable -- the pool is full of held modules, or modules in front of it in the queue
    wait for a slot -- is the call on which the reference spins forever; here it raises."""

    def __init__(self, keys, n_slots, on_demand=False):
        self.queue, self.n_slots, self.on_demand = list(keys), n_slots, on_demand
        self.resident, self.held, self.calls, self.synced = [], set(), [], True

    def _pump(self):
        while not self.on_demand and len(self.resident) < self.n_slots and self.queue[0] not in self.resident:
            self.resident.append(self.queue[0])
            self.queue.append(self.queue.pop(0))

    def fetch(self, keys):
        for key in keys:
            if key not in self.resident:
                assert len(self.resident) < self.n_slots, f"no free slot for {key}"
                self.resident.append(key)

    def get_weights(self, key):
        self._pump()
        assert key in self.resident, f"get_weights({key}) would block forever: pool holds {self.resident}"
        self.held.add(key)
        assert len(self.held) <= self.n_slots
        self.calls.append(("get", key))
        return {n + ".weight": torch.zeros(2, 2) for n in ("gate_proj", "up_proj", "down_proj")}

    def free_weights_buffer(self, key):
        assert self.synced, "slot released while kernels that read it may still run"
        self.held.remove(key); self.resident.remove(key)
        self.calls.append(("free", key))

    def clear_expert_buffer(self, layer_idx, expert_idx):
        self.calls.append(("clear", layer_idx, expert_idx))


class _Wrapped(torch.nn.Module):
    names = ("gate_proj", "up_proj", "down_proj")

    def __init__(self, eng, L, e, engine_config=None):
        super().__init__()
        self.module = self
        for n in self.names:
            setattr(self, n, torch.nn.Linear(2, 2, bias=False))
        self.layer_idx, self.expert_idx, self.core_engine, self.get_weights = L, e, eng, True
        self.expert_weights_idx = f"routed_expert_{L}_{e}"
        self.weight_dequant_scale = None
        if engine_config is not None:
            self.engine_config = engine_config


def _engine_config(prefill, decoding):
    from types import SimpleNamespace as NS
    return NS(GPU_Buffer_Config=NS(num_prefill_module_buffer={"routed_expert": prefill, "shared_expert": 1},
                                   num_decoding_module_buffer={"routed_expert": decoding, "shared_expert": 1}))


@pytest.mark.parametrize("E,slots", [(64, 20), (8, 8), (8, 3), (5, 1), (256, 20)])
def test_engine_pool_smaller_than_the_layer_runs_in_waves(E, slots):
    """The reference's prefill pool holds 20 routed experts (deepseekv3_initializer.py:912-916) and
    its get_weights blocks until the copy worker delivers (GPU_Weight_Buffer.cpp:171-246): the
    block must never hold more than the pool, must ask for experts in delivery order, and must
    drain the stream before it frees a slot of an engine that does not order releases itself."""
    from moe_gen_amd import block
    L = 5
    keys = [f"routed_expert_{L}_{e}" for e in range(E)] + [f"routed_expert_{L + 1}_{e}" for e in range(E)]
    eng = _SlotLimitedEngine(keys, slots)
    experts = [_Wrapped(eng, L, e, _engine_config(slots, 4 * slots)) for e in range(E)]
    assert block.pool_size(experts[0]) == slots
    counts = [(7 * e) % 5 for e in range(E)]
    launches = []

    def launch(rows, a, b, n_rows):
        assert len(rows) == b - a and all(f"routed_expert_{L}_{e}" in eng.held for e in range(a, b))
        launches.append((a, b, n_rows))
        eng.synced = False                                   # kernels reading the slots are now queued

    def stream_wait():
        eng.synced = True

    block.staged_experts_forward(experts, launch, counts, stream_wait=stream_wait)
    step = slots if E <= slots else max(1, slots // 2)       # half the pool per wave: the other half is being copied
    assert [a for a, _, _ in launches] == list(range(0, E, step))
    assert launches[-1][1] == E and all(b - a <= step for a, b, _ in launches)
    assert [n for _, _, n in launches] == [sum(counts[a:b]) for a, b, _ in launches]
    assert not eng.held and eng.calls[0] == ("clear", L, 0)
    gets = [c[1] for c in eng.calls if c[0] == "get"]
    assert gets == keys[:E] and sorted(c[1] for c in eng.calls if c[0] == "free") == sorted(gets)
    if E > slots:
        with pytest.raises(RuntimeError, match="more than one wave"):
            block.staged_experts_forward(experts, launch, None, stream_wait=stream_wait)


def test_engine_phase_and_unknown_pool():
    from moe_gen_amd import block
    eng = _SlotLimitedEngine([f"routed_expert_0_{e}" for e in range(4)], 4)

    class DecodingWrapped(_Wrapped):
        phase = "decoding"

    assert block.pool_size(DecodingWrapped(eng, 0, 0, _engine_config(2, 4))) == 4
    assert block.pool_size(_Wrapped(eng, 0, 0, _engine_config(2, 4))) == 2
    assert block.pool_size(_Wrapped(eng, 0, 0)) == 1          # nothing known: one at a time, as Wrapper.py:475-521
    assert block.expert_waves(2, 2) == [(0, 2, [0, 1])]                                   # fits the pool: one wave
    assert block.expert_waves(5, 4) == [(0, 2, [0, 1]), (2, 4, [2, 3]), (4, 5, [4])]     # else half the pool per wave
    assert block.expert_waves(3, 1) == [(0, 1, [0]), (1, 2, [1]), (2, 3, [2])]
    assert block.expert_waves(9, 4, hot=[7, 1, 4, 8, 2]) == [(1, 3, [1, 2]), (4, 8, [4, 7]), (8, 9, [8])]


def test_on_demand_waves_fetch_only_experts_with_tokens():
    from moe_gen_amd import block
    E, slots, L = 12, 3, 2
    eng = _SlotLimitedEngine([f"routed_expert_{L}_{e}" for e in range(E)], slots, on_demand=True)
    eng.pool_size = lambda module_type: slots
    eng.stream_ordered_release = True
    experts = [_Wrapped(eng, L, e) for e in range(E)]
    counts = [0, 3, 0, 0, 9, 1, 0, 2, 0, 0, 5, 0]
    launches = []
    block.staged_experts_forward(experts, lambda rows, a, b, n: launches.append((a, b, n)), counts, on_demand=True)
    assert launches == [(1, 2, 3), (4, 5, 9), (5, 6, 1), (7, 8, 2), (10, 11, 5)]     # 5 hot experts, 3 slots: one per wave
    assert [c[1] for c in eng.calls if c[0] == "get"] == [f"routed_expert_{L}_{e}" for e in (1, 4, 5, 7, 10)]
    eng.calls.clear()
    few = [0, 0, 4, 0, 0, 0, 0, 0, 6, 0, 0, 0]                # fits the pool: one wave, busiest first
    launches.clear()
    block.staged_experts_forward(experts, lambda rows, a, b, n: launches.append((a, b, n)), few, on_demand=True)
    assert launches == [(2, 9, 10)] and not eng.held


@pytest.mark.parametrize("slots", [1, 2, 3])
def test_on_demand_waves_with_a_tiny_pool(slots):
    """More hot experts than slots: a wave is half the pool and the next wave is asked for while this
    one is multiplied -- except with a single slot, which has no other half: its next copy is asked
    for only after the slot has been let go.  Against the stand-in engine and against the library's
    Stager (host backend), whose fetch fails when no slot is free."""
    from moe_gen_amd import Stager, block
    E, L = 7, 3
    counts = [2, 0, 5, 1, 0, 3, 4]
    hot = [e for e in range(E) if counts[e]]
    eng = _SlotLimitedEngine([f"routed_expert_{L}_{e}" for e in range(E)], slots, on_demand=True)
    eng.pool_size = lambda module_type: slots
    eng.stream_ordered_release = True
    launches = []
    block.staged_experts_forward([_Wrapped(eng, L, e) for e in range(E)], lambda rows, a, b, n: launches.append((a, b, n)),
                                 counts, on_demand=True)
    assert sum(n for _, _, n in launches) == sum(counts) and not eng.held and not eng.resident
    assert [c[1] for c in eng.calls if c[0] == "get"] == [f"routed_expert_{L}_{e}" for e in hot]

    shapes = {"routed_expert": {f"{n}.weight": ((2, 2), torch.float32) for n in _Wrapped.names}}
    st = Stager(shapes, {"routed_expert": slots}, backend="host", model_type="mixtral", num_hidden_layers=L + 1,
                num_local_experts=E)
    st.set_policy("routed_expert", "on_demand")
    for e in range(E):
        st.add_module(f"routed_expert_{L}_{e}", "routed_expert",
                      {f"{n}.weight": torch.full((2, 2), float(e)) for n in _Wrapped.names})
    seen = []

    def launch(rows, a, b, n):
        for e in range(a, b):
            if counts[e]:
                seen.append((e, float(rows[e - a][0][0, 0])))          # the gate matrix handed out for expert e

    for rep in range(2):
        seen.clear()
        block.staged_experts_forward([_Wrapped(st, L, e) for e in range(E)], launch, counts, on_demand=True)
        assert seen == [(e, float(e)) for e in hot]
        assert st.stats()[0] == (rep + 1) * len(hot)
        assert not any(st.resident(f"routed_expert_{L}_{e}") for e in range(E))


def test_layer_with_resident_and_engine_backed_experts():
    """The reference sets get_weights expert by expert (Mixtral_Initializer.py:761-787,
    deepseekv3_initializer.py:1259-1266): experts outside the copy task keep their weights.  Only the
    engine-backed ones count against the pool, every expert lands in exactly one wave, and a resident
    expert is never asked of the engine."""
    from moe_gen_amd import block
    E, slots, L = 9, 4, 2
    backed = [1, 2, 4, 5, 6, 8]
    eng = _SlotLimitedEngine([f"routed_expert_{L}_{e}" for e in backed], slots)
    experts = [_Wrapped(eng, L, e, _engine_config(slots, slots)) for e in range(E)]
    for e in range(E):
        if e not in backed:
            experts[e].get_weights = False
            experts[e].gate_proj.weight.data.fill_(100.0 + e)
    counts = [3, 1, 0, 2, 5, 1, 1, 4, 2]
    covered, launches = [], []

    def launch(rows, a, b, n):
        launches.append((a, b, n))
        for e in range(a, b):
            covered.append(e)
            if e in backed:
                assert f"routed_expert_{L}_{e}" in eng.held
            else:
                assert float(rows[e - a][0][0, 0]) == 100.0 + e       # its own resident gate matrix
        eng.synced = False

    def stream_wait():
        eng.synced = True

    block.staged_experts_forward(experts, launch, counts, stream_wait=stream_wait)
    assert covered == list(range(E)) and sum(n for _, _, n in launches) == sum(counts)
    assert [c[1] for c in eng.calls if c[0] == "get"] == [f"routed_expert_{L}_{e}" for e in backed]
    assert not eng.held
    assert block.expert_waves(9, 4, backed=backed) == [(0, 4, [1, 2]), (4, 6, [4, 5]), (6, 9, [6, 8])]
    assert block.expert_waves(9, 8, backed=backed) == [(0, 9, backed)]
    assert block.expert_waves(4, 2, hot=[], backed=[1, 3]) == [(0, 4, [])]
    with pytest.raises(RuntimeError, match="no expert of the layer"):
        for ex in experts:
            ex.get_weights = False
        block.staged_experts_forward(experts, launch, counts)
