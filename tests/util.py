"""Helpers shared by the tests: torch <-> raw-bit numpy views and oracle-side weight views."""
import numpy as np
import torch

from oracle import oracle as O


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> uint16 bit array; fp8 tensor -> uint8; others -> numpy."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).numpy()
    return t.numpy()


def bf16_tensor(a: np.ndarray, device="cpu") -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16).to(device)


def weight_f32(lin) -> np.ndarray:
    """fp32 view of a Linear's weight as the kernels see it: bf16 values, or the block
    dequantisation bf16(f32(q) * scale) computed by the ORACLE for fp8 weights."""
    w = lin.weight.data
    if w.dtype == torch.float8_e4m3fn:
        return O.bf16_to_f32(O.dequant_block(bits(w), lin.weight_scale_inv.data.cpu().numpy()))
    return O.bf16_to_f32(bits(w))


def oracle_weights(blk, family: str) -> O.LayerWeights:
    gate = bits(blk.gate.weight.data)
    bias = blk.gate.e_score_correction_bias.data.cpu().numpy() if family == "v3" else None
    wg, wu, wd = [], [], []
    for ex in blk.experts:
        g, u, d = ex.projections()
        wg.append(weight_f32(g)); wu.append(weight_f32(u)); wd.append(weight_f32(d))
    shared = None
    if family != "mixtral" and getattr(blk.config, "n_shared_experts", None):
        shared = tuple(weight_f32(p) for p in blk.shared_experts.projections())
    return O.LayerWeights(gate, bias, wg, wu, wd, shared)


def oracle_spec(w) -> O.RouterSpec:
    if w.family == "v3":
        return O.RouterSpec.deepseek_v3(w.E, w.k, w.n_group, w.topk_group, w.norm, w.scale)
    if w.family == "v2":
        return O.RouterSpec.deepseek_v2(w.E, w.k, w.method, w.n_group, w.topk_group, w.norm, w.scale)
    return O.RouterSpec.mixtral(w.E, w.k)


def rel_max(y, ref) -> float:
    y = np.asarray(y, np.float64); ref = np.asarray(ref, np.float64)
    return float(np.abs(y - ref).max() / max(np.abs(ref).max(), 1e-30))


def rel_rms(y, ref) -> float:
    y = np.asarray(y, np.float64); ref = np.asarray(ref, np.float64)
    return float(np.sqrt(((y - ref) ** 2).mean()) / max(np.sqrt((ref ** 2).mean()), 1e-30))
