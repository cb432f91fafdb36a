"""MI355X-native MoE layer (router, dispatch, grouped SwiGLU experts, combine, weight
staging) behind the module surface of MoE-Gen's MoE blocks."""
from . import ops  # noqa: F401
from .arena import Arena, ArenaIndex  # noqa: F401
from .block import norm_moe_residual  # noqa: F401
from .config import DeepseekV2Config, DeepseekV3Config, MixtralConfig  # noqa: F401
from .deepseek_v2 import DeepseekV2MLP, DeepseekV2MoE  # noqa: F401
from .deepseek_v3 import DeepseekV3MLP, DeepseekV3MoE, MoEGate  # noqa: F401
from .mixtral import MixtralBlockSparseTop2MLP, MixtralSparseMoeBlock  # noqa: F401
from .stager import StagedExpert, Stager  # noqa: F401
