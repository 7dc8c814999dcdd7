from .fused_moe import (fused_experts, fused_experts_gated, fused_experts_normed, fused_topk, gate_topk,  # noqa: F401
                        norm_gate_topk)
from .mixtral_block import MixtralMoE, PostAttentionMoE, ReplicatedLinear  # noqa: F401
from .mixtral_moe import FusedMoE  # noqa: F401
from .moe_align_block_size import moe_align_block_size  # noqa: F401
