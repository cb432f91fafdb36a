"""The five synthetic MoE-layer workloads of the benchmark (model-shaped, random weights)
and their generators.  Inputs are drawn in fp32 from a seeded torch generator and rounded to
bf16, so that every consumer (GPU path, CPU baseline, oracle) sees the same bits.

Per-expert "Zipf logit bias": the reference gate has no bias term
(modeling_deepseek_v3.py:486-488), so load skew is expressed through the gate's own
surface: hidden[:, 0] = 1 and W_gate[e, 0] = b_e with b_e = ln p_pi(e) - mean(ln p),
p_r ~ r^-s, pi a seeded permutation of the experts.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace

import torch
from torch import nn

from .block import attach_fp8_weight
from .config import DeepseekV2Config, DeepseekV3Config, MixtralConfig
from .deepseek_v2 import DeepseekV2MoE
from .deepseek_v3 import DeepseekV3MoE
from .mixtral import MixtralSparseMoeBlock


@dataclass(frozen=True)
class Workload:
    name: str
    family: str            # "v2" | "v3" | "mixtral"
    n: int                 # tokens
    h: int
    E: int
    k: int
    I: int
    S: int = 0             # shared experts
    method: str = "greedy"
    n_group: int = 1
    topk_group: int = 1
    norm: bool = False
    scale: float = 1.0
    seed: int = 0
    zipf: float | None = None
    fp8: bool = False
    seq: int = 512         # tokens are presented as [n/seq, seq, h]

    def scaled(self, **kw) -> "Workload":
        return replace(self, **kw)

    @property
    def routed_flop(self) -> float:
        return 6.0 * self.n * self.k * self.h * self.I

    @property
    def shared_flop(self) -> float:
        return 6.0 * self.n * self.h * self.S * self.I

    @property
    def router_bytes(self) -> float:
        return 2.0 * self.n * self.h + 2.0 * self.E * self.h + 8.0 * self.n * self.k + 4.0 * self.E

    @property
    def dispatch_bytes(self) -> float:
        return 4.0 * self.n * self.k + 2.0 * (2.0 * self.n * self.k * self.h)

    @property
    def combine_bytes(self) -> float:
        return (2.0 * self.n * self.k * self.h + 4.0 * self.n * self.k
                + (2.0 * self.n * self.h if self.S > 0 else 0.0) + 2.0 * self.n * self.h)


WORKLOADS = {
    "deepseek_v2_lite": Workload("deepseek_v2_lite", "v2", 4096, 2048, 64, 6, 1408, S=2, method="greedy",
                                 scale=1.0, seed=0, zipf=1.1),
    "mixtral_8x7b": Workload("mixtral_8x7b", "mixtral", 16384, 4096, 8, 2, 14336, norm=True, seed=1),
    "mixtral_8x22b": Workload("mixtral_8x22b", "mixtral", 8192, 6144, 8, 2, 16384, norm=True, seed=2, zipf=1.2),
    "mixtral_8x22b_decode": Workload("mixtral_8x22b_decode", "mixtral", 256, 6144, 8, 2, 16384, norm=True, seed=2,
                                     zipf=1.2, seq=1),
    "deepseek_v2_236b": Workload("deepseek_v2_236b", "v2", 32768, 5120, 160, 6, 1536, S=2,
                                 method="group_limited_greedy", n_group=8, topk_group=3, scale=16.0, seed=3,
                                 zipf=1.1),
    "deepseek_v3_w8a16": Workload("deepseek_v3_w8a16", "v3", 65536, 7168, 256, 8, 2048, S=1, method="noaux_tc",
                                  n_group=8, topk_group=4, norm=True, scale=2.5, seed=4, fp8=True),
}


def _gen(seed: int, device) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def hidden_states(w: Workload, device="cpu") -> torch.Tensor:
    """bf16 [n/seq, seq, h] ~ N(0,1) (column 0 set to 1 when the workload has a Zipf bias)."""
    x = torch.randn((w.n, w.h), generator=_gen(w.seed, device), device=device, dtype=torch.float32)
    if w.zipf is not None:
        x[:, 0] = 1.0
    seq = w.seq if w.n % w.seq == 0 else 1
    return x.to(torch.bfloat16).view(w.n // seq, seq, w.h)


def gate_weight(w: Workload, device="cpu") -> torch.Tensor:
    g = _gen(w.seed + 7919, device)
    W = torch.randn((w.E, w.h), generator=g, device=device, dtype=torch.float32) * 0.02
    if w.zipf is not None:
        ranks = torch.arange(1, w.E + 1, dtype=torch.float64)
        lp = -w.zipf * torch.log(ranks)
        lp = lp - torch.logsumexp(lp, 0)
        pi = torch.randperm(w.E, generator=_gen(w.seed + 104729, "cpu"))
        b = (lp[pi] - lp.mean()).to(torch.float32)
        W[:, 0] = b.to(device)
    return W.to(torch.bfloat16)


def score_bias(w: Workload, device="cpu") -> torch.Tensor:
    return torch.randn((w.E,), generator=_gen(w.seed + 15485863, device), device=device, dtype=torch.float32) * 0.01


def quantize_fp8_block128(x: torch.Tensor):
    """per_block_cast_to_fp8 (deepseekv3_initializer.py:191-205): q = fp8(x * 448/amax),
    scale = amax/448 with amax = clamp(max|x| of the 128x128 block, 1e-4)."""
    m, n = x.shape
    mp, npad = math.ceil(m / 128) * 128, math.ceil(n / 128) * 128
    xp = torch.zeros((mp, npad), dtype=x.dtype, device=x.device)
    xp[:m, :n] = x
    v = xp.view(mp // 128, 128, npad // 128, 128)
    amax = v.abs().float().amax(dim=(1, 3), keepdim=True).clamp(1e-4)
    q = (v * (448.0 / amax)).to(torch.float8_e4m3fn).view(mp, npad)[:m, :n].contiguous()
    return q, (amax / 448.0).view(mp // 128, npad // 128).contiguous()


def expert_weights(w: Workload, e: int, device="cpu", inter: int | None = None):
    """(gate [I,h], up [I,h], down [h,I]) of expert e (e == E: the shared expert, I = S*I), drawn
    N(0, 0.02) from seed*10^6 + e.  bf16 tensors, or (fp8, fp32 scale) pairs when w.fp8."""
    I = inter if inter is not None else w.I
    g = _gen(w.seed * 1_000_000 + e, device)
    mats = []
    for shape in ((I, w.h), (I, w.h), (w.h, I)):
        m = torch.randn(shape, generator=g, device=device, dtype=torch.float32) * 0.02
        mats.append(quantize_fp8_block128(m) if w.fp8 else m.to(torch.bfloat16))
    return mats


def _assign(mlp, mats, fp8: bool):
    for lin, m in zip(mlp.projections(), mats):
        if fp8:
            attach_fp8_weight(lin, m[0], m[1])
        else:
            lin.weight = nn.Parameter(m, requires_grad=False)


def build_block(w: Workload, device="cuda", gen_device=None):
    """The MoE block of workload `w` with its synthetic weights on `device`.  Modules are created
    on the meta device (no 45 GB of throw-away fp32 initialisation) and then given real tensors,
    the way MoE-Gen assigns `param.data` after construction (deepseekv3_initializer.py:1011-1021)."""
    gd = gen_device or device
    if w.family == "v3":
        cfg = DeepseekV3Config(hidden_size=w.h, moe_intermediate_size=w.I, n_shared_experts=w.S or None,
                               n_routed_experts=w.E, routed_scaling_factor=w.scale, n_group=w.n_group,
                               topk_group=w.topk_group, num_experts_per_tok=w.k, norm_topk_prob=w.norm)
        with torch.device("meta"):
            blk = DeepseekV3MoE(cfg)
    elif w.family == "v2":
        cfg = DeepseekV2Config(hidden_size=w.h, moe_intermediate_size=w.I, n_shared_experts=w.S or None,
                               n_routed_experts=w.E, routed_scaling_factor=w.scale, topk_method=w.method,
                               n_group=w.n_group, topk_group=w.topk_group, num_experts_per_tok=w.k,
                               norm_topk_prob=w.norm)
        with torch.device("meta"):
            blk = DeepseekV2MoE(cfg)
    else:
        cfg = MixtralConfig(hidden_size=w.h, intermediate_size=w.I, num_local_experts=w.E, num_experts_per_tok=w.k)
        with torch.device("meta"):
            blk = MixtralSparseMoeBlock(cfg)
    blk.eval()
    gw = gate_weight(w, gd).to(device)
    blk.gate.weight = nn.Parameter(gw, requires_grad=False)
    if w.family == "v3":
        blk.gate.e_score_correction_bias = nn.Parameter(score_bias(w, gd).to(device), requires_grad=False)

    def to_dev(mats):
        return [tuple(t.to(device) for t in m) if isinstance(m, tuple) else m.to(device) for m in mats]

    for e in range(w.E):
        _assign(blk.experts[e], to_dev(expert_weights(w, e, gd)), w.fp8)
    if w.S and w.family != "mixtral":
        _assign(blk.shared_experts, to_dev(expert_weights(w, w.E, gd, inter=w.S * w.I)), w.fp8)
    return blk
