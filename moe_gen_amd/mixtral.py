"""Mixtral sparse MoE block with the surface of transformers-4.42.0's MixtralSparseMoeBlock /
MixtralBlockSparseTop2MLP, the classes MoE-Gen imports (Mixtral_Initializer.py:31-35) and whose
experts it addresses as block_sparse_moe.experts[i].{w1,w2,w3} (:691-716)."""
from __future__ import annotations

import torch
from torch import nn

from . import ops
from .block import SwiGLUMLP, _require_silu, moe_forward


class MixtralBlockSparseTop2MLP(SwiGLUMLP):
    """w2(silu(w1 x) * w3 x): w1 = gate [ffn,h], w3 = up [ffn,h], w2 = down [h,ffn]
    (shapes: Mixtral_Initializer.py:398-402)."""

    names = ("w1", "w3", "w2")

    def __init__(self, config):
        _require_silu(config)
        super().__init__(config.hidden_size, config.intermediate_size)
        self.ffn_dim = config.intermediate_size
        self.hidden_dim = config.hidden_size


class MixtralSparseMoeBlock(nn.Module):
    """bf16 gate Linear -> fp32 softmax -> top-k -> renormalise -> bf16 weights; experts in
    index order accumulate into a bf16 result.  Returns (hidden_states, router_logits)."""

    def __init__(self, config):
        super().__init__()
        self.hidden_dim = config.hidden_size
        self.ffn_dim = config.intermediate_size
        self.num_experts = config.num_local_experts
        self.top_k = config.num_experts_per_tok
        self.gate = nn.Linear(self.hidden_dim, self.num_experts, bias=False)
        self.experts = nn.ModuleList([MixtralBlockSparseTop2MLP(config) for _ in range(self.num_experts)])
        self.jitter_noise = getattr(config, "router_jitter_noise", 0.0)

    @torch.no_grad()
    def forward(self, hidden_states):
        if self.training:
            raise NotImplementedError("inference only")
        spec = ops.RouterSpec(self.num_experts, self.top_k, "softmax", "greedy", 1, 1, True, 0, 1.0, 0.0, True, True)
        out, logits = moe_forward(self, hidden_states, spec, self.gate.weight, None, self.experts, None,
                                  ops.COMBINE_BF16_SEQ, want_logits=True)
        return out, logits.to(hidden_states.dtype)
