"""Routing / shape hyper-parameters under the names the reference's HF configs use
(configuration_deepseek_v3.py:137-180, configuration_deepseek_v2.py:135-177, MixtralConfig).
Any object carrying these attributes (an HF config included) can be passed to the blocks;
these dataclasses exist so the blocks can be built without transformers."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class DeepseekV3Config:
    hidden_size: int = 7168
    intermediate_size: int = 18432
    moe_intermediate_size: int = 2048
    n_shared_experts: int | None = 1
    n_routed_experts: int = 256
    ep_size: int = 1
    routed_scaling_factor: float = 2.5
    topk_method: str = "noaux_tc"
    n_group: int = 8
    topk_group: int = 4
    num_experts_per_tok: int = 8
    norm_topk_prob: bool = True
    scoring_func: str = "sigmoid"
    seq_aux: bool = True
    hidden_act: str = "silu"
    model_type: str = "deepseek_v3"


@dataclass
class DeepseekV2Config:
    hidden_size: int = 4096
    intermediate_size: int = 11008
    moe_intermediate_size: int = 1408
    n_shared_experts: int | None = None
    n_routed_experts: int | None = None
    ep_size: int = 1
    routed_scaling_factor: float = 1.0
    topk_method: str = "greedy"
    n_group: int | None = None
    topk_group: int | None = None
    num_experts_per_tok: int | None = None
    norm_topk_prob: bool = False
    scoring_func: str = "softmax"
    aux_loss_alpha: float = 0.001
    seq_aux: bool = True
    hidden_act: str = "silu"
    model_type: str = "deepseek_v2"


@dataclass
class MixtralConfig:
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_local_experts: int = 8
    num_experts_per_tok: int = 2
    hidden_act: str = "silu"
    router_jitter_noise: float = 0.0
    model_type: str = "mixtral"
