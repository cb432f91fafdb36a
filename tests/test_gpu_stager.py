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


class FakeCoreEngine:
    """Stands in for MoE-Gen's pybind `core_engine` (MoE_Gen_Binding.cpp:45-65): hands out device
    tensors by module key and records the protocol calls."""

    def __init__(self, weights):
        self.weights, self.calls, self.held = weights, [], set()

    def get_weights(self, key):
        self.calls.append(("get", key)); self.held.add(key)
        return self.weights[key]

    def free_weights_buffer(self, key):
        self.calls.append(("free", key)); self.held.remove(key)

    def clear_expert_buffer(self, layer_idx, expert_idx):
        self.calls.append(("clear", layer_idx, expert_idx))


class ExpertWrapperLike(torch.nn.Module):
    """Attribute-for-attribute what the reference's Expert_Wrapper exposes (Wrapper.py:437-468)."""

    def __init__(self, module, layer_idx, expert_idx, core_engine, scales):
        super().__init__()
        self.module, self.layer_idx, self.expert_idx = module, layer_idx, expert_idx
        self.core_engine, self.get_weights, self.weight_dequant_scale = core_engine, True, scales
        self.expert_weights_idx = (f"routed_expert_{layer_idx}_{expert_idx}" if expert_idx >= 0
                                   else f"shared_expert_{layer_idx}")


@pytest.mark.parametrize("name", ["deepseek_v3_w8a16", "deepseek_v2_236b"])
def test_block_with_engine_backed_experts(name):
    """The block fed through MoE-Gen's expert-wrapper protocol gives the same bits as with resident
    weights, and calls get_weights / free_weights_buffer once per expert."""
    from moe_gen_amd import synthetic
    w = synthetic.WORKLOADS[name].scaled(n=256, h=512, I=256, seq=64)
    blk = synthetic.build_block(w, device="cuda", gen_device="cpu")
    x = synthetic.hidden_states(w, "cpu").cuda()
    ref = blk(x).clone()
    names = blk.experts[0].names
    L = 7
    weights, wrapped = {}, []

    def detach(mlp, key):
        weights[key] = {f"{n}.weight": getattr(mlp, n).weight.data.clone() for n in names}
        scales = {f"{n}.weight_scale_inv": getattr(mlp, n).weight_scale_inv.data for n in names} if w.fp8 else None
        for n in names:                                   # placeholders, as MoE-Gen leaves them
            getattr(mlp, n).weight.data = torch.zeros(1, dtype=torch.bfloat16, device="cuda")
        return scales

    eng = FakeCoreEngine(weights)
    for e, ex in enumerate(blk.experts):
        wrapped.append(ExpertWrapperLike(ex, L, e, eng, detach(ex, f"routed_expert_{L}_{e}")))
    blk.experts = torch.nn.ModuleList(wrapped)
    blk.shared_experts = ExpertWrapperLike(blk.shared_experts, L, -1, eng, detach(blk.shared_experts, f"shared_expert_{L}"))
    out = blk(x)
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
    gets = [c[1] for c in eng.calls if c[0] == "get"]
    frees = [c[1] for c in eng.calls if c[0] == "free"]
    assert sorted(gets) == sorted(frees) == sorted(weights) and not eng.held
    assert ("clear", L, 0) in eng.calls


def test_block_with_library_stager():
    """Same, with the library's own Stager delivering fp8 experts from pinned host memory."""
    from moe_gen_amd import StagedExpert, Stager, synthetic
    w = synthetic.WORKLOADS["deepseek_v3_w8a16"].scaled(n=256, h=512, I=256, E=16, n_group=4, topk_group=2, k=4, seq=64)
    blk = synthetic.build_block(w, device="cuda", gen_device="cpu")
    x = synthetic.hidden_states(w, "cpu").cuda()
    ref = blk(x).clone()
    names = blk.experts[0].names
    fp8 = torch.float8_e4m3fn
    shapes = {"routed_expert": {f"{n}.weight": (tuple(getattr(blk.experts[0], n).weight.shape), fp8) for n in names},
              "shared_expert": {f"{n}.weight": (tuple(getattr(blk.shared_experts, n).weight.shape), fp8) for n in names}}
    st = Stager(shapes, {"routed_expert": w.E, "shared_expert": 1}, model_type="deepseek_v3", num_hidden_layers=8,
                num_local_experts=w.E)
    L = 5
    wrapped = []
    for e, ex in enumerate(blk.experts):
        st.add_module(f"routed_expert_{L}_{e}", "routed_expert",
                      {f"{n}.weight": getattr(ex, n).weight.data.cpu().pin_memory() for n in names})
        wrapped.append(StagedExpert(ex, L, e, st, {f"{n}.weight_scale_inv": getattr(ex, n).weight_scale_inv.data for n in names}))
    sh = blk.shared_experts
    st.add_module(f"shared_expert_{L}", "shared_expert", {f"{n}.weight": getattr(sh, n).weight.data.cpu().pin_memory() for n in names})
    blk.experts = torch.nn.ModuleList(wrapped)
    blk.shared_experts = StagedExpert(sh, L, -1, st, {f"{n}.weight_scale_inv": getattr(sh, n).weight_scale_inv.data for n in names})
    for _ in range(3):                                    # slots are recycled between calls
        out = blk(x)
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
    assert st.stats()[0] >= 3 * (w.E + 1)
    st.close()


def test_block_with_routing_aware_staging():
    """With per-expert token counts on the host, only experts that received tokens are staged
    (busiest first); the output is bit-identical to resident weights and the copy count equals the
    number of such experts.  The reference's worker copies every expert of the layer."""
    from moe_gen_amd import StagedExpert, Stager, synthetic
    w = synthetic.WORKLOADS["deepseek_v3_w8a16"].scaled(n=24, h=512, I=256, E=64, n_group=8, topk_group=4, k=4, seq=8)
    blk = synthetic.build_block(w, device="cuda", gen_device="cpu")
    x = synthetic.hidden_states(w, "cpu").cuda()
    ref = blk(x).clone()
    used = int((blk.last_counts > 0).sum())
    assert 0 < used < w.E                                  # 24 tokens x 4 slots cannot reach all 64 experts
    names = blk.experts[0].names
    fp8 = torch.float8_e4m3fn
    shapes = {"routed_expert": {f"{n}.weight": (tuple(getattr(blk.experts[0], n).weight.shape), fp8) for n in names},
              "shared_expert": {f"{n}.weight": (tuple(getattr(blk.shared_experts, n).weight.shape), fp8) for n in names}}
    st = Stager(shapes, {"routed_expert": w.E, "shared_expert": 1}, model_type="deepseek_v3", num_hidden_layers=8,
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
