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
