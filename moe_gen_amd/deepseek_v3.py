"""DeepSeek-V3 / R1 MoE layer with the reference's module surface
(modeling_deepseek_v3.py:439-711): DeepseekV3MLP, MoEGate, DeepseekV3MoE."""
from __future__ import annotations

import math

import torch
from torch import nn

from . import ops
from .block import SwiGLUMLP, _require_silu, moe_forward


class DeepseekV3MLP(SwiGLUMLP):
    """modeling_deepseek_v3.py:439-467."""

    def __init__(self, config, hidden_size=None, intermediate_size=None):
        _require_silu(config)
        super().__init__(config.hidden_size if hidden_size is None else hidden_size,
                         config.intermediate_size if intermediate_size is None else intermediate_size)
        self.config = config


def _spec(gate) -> ops.RouterSpec:
    if gate.scoring_func != "sigmoid":
        raise NotImplementedError(f"insupportable scoring function for MoE gating: {gate.scoring_func}")
    if gate.topk_method != "noaux_tc":
        raise NotImplementedError(f"insupportable TopK function for MoE gating: {gate.topk_method}")
    return ops.RouterSpec(gate.n_routed_experts, gate.top_k, "sigmoid", "noaux_tc", gate.n_group, gate.topk_group,
                          bool(gate.norm_topk_prob), 2, float(gate.routed_scaling_factor), 1e-20)


class MoEGate(nn.Module):
    """modeling_deepseek_v3.py:470-561: sigmoid scores + e_score_correction_bias, group-limited
    top-k (group score = sum of its two best), renormalisation, routed scaling."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.top_k = config.num_experts_per_tok
        self.n_routed_experts = config.n_routed_experts
        self.routed_scaling_factor = config.routed_scaling_factor
        self.scoring_func = config.scoring_func
        self.seq_aux = getattr(config, "seq_aux", True)
        self.topk_method = config.topk_method
        self.n_group = config.n_group
        self.topk_group = config.topk_group
        self.norm_topk_prob = config.norm_topk_prob
        self.gating_dim = config.hidden_size
        self.weight = nn.Parameter(torch.empty((self.n_routed_experts, self.gating_dim)))
        if self.topk_method == "noaux_tc":
            self.e_score_correction_bias = nn.Parameter(torch.empty((self.n_routed_experts)))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if hasattr(self, "e_score_correction_bias"):
            nn.init.zeros_(self.e_score_correction_bias)

    @torch.no_grad()
    def forward(self, hidden_states):
        """-> (topk_idx int64 [n,k], topk_weight fp32 [n,k]); slots in descending score."""
        assert not self.training
        from .block import _gate_weight_bf16
        spec = _spec(self)
        h = hidden_states.shape[-1]
        x = hidden_states.reshape(-1, h)
        cache = self.__dict__.setdefault("_moe_cache", {})
        idx, w, _ = ops.router(x.contiguous(), _gate_weight_bf16(self.weight, cache),
                               self.e_score_correction_bias.data.to(torch.float32), spec)
        return idx.to(torch.int64), w


class DeepseekV3MoE(nn.Module):
    """modeling_deepseek_v3.py:564-711: routed experts + shared experts, inference path."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.num_experts_per_tok = config.num_experts_per_tok
        if getattr(config, "ep_size", 1) > 1:
            raise NotImplementedError("expert parallelism (ep_size > 1) is outside this single-GPU build")
        self.ep_size, self.experts_per_rank, self.ep_rank = 1, config.n_routed_experts, 0
        self.experts = nn.ModuleList(
            [DeepseekV3MLP(config, intermediate_size=config.moe_intermediate_size)
             for _ in range(config.n_routed_experts)])
        self.gate = MoEGate(config)
        if config.n_shared_experts is not None:
            self.shared_experts = DeepseekV3MLP(
                config=config, intermediate_size=config.moe_intermediate_size * config.n_shared_experts)

    @torch.no_grad()
    def forward(self, hidden_states):
        if self.training:
            raise NotImplementedError("inference only (the reference's moe_infer path)")
        shared = self.shared_experts if self.config.n_shared_experts is not None else None
        out, _ = moe_forward(self, hidden_states, _spec(self.gate), self.gate.weight,
                             self.gate.e_score_correction_bias, self.experts, shared, ops.COMBINE_F32)
        return out
