"""MI355X-native Mixtral MoE layer: the hot path of electrock-infer rebuilt as
hand-written gfx950 HIP kernels behind the reference's own layer call
(``FusedMoE``) and op names (``_C.topk_softmax``, ``_C.moe_align_block_size``,
``_C.silu_and_mul``, ``_C.moe_sum``)."""
from . import _C  # noqa: F401
from .layers.layernorm import RMSNorm  # noqa: F401
from .layers.moe.fused_moe import (fused_experts, fused_experts_gated, fused_experts_normed, fused_topk,  # noqa: F401
                                   gate_topk, norm_gate_topk)
from .layers.moe.mixtral_block import MixtralMoE, PostAttentionMoE  # noqa: F401
from .layers.moe.mixtral_moe import FusedMoE  # noqa: F401
from .layers.moe.moe_align_block_size import moe_align_block_size  # noqa: F401

__all__ = ["_C", "FusedMoE", "MixtralMoE", "PostAttentionMoE", "RMSNorm", "fused_experts", "fused_experts_gated",
           "fused_experts_normed", "fused_topk", "gate_topk", "norm_gate_topk", "moe_align_block_size"]
