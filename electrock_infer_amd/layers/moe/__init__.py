from .fused_moe import fused_experts, fused_experts_gated, fused_topk, gate_topk  # noqa: F401
from .mixtral_block import MixtralMoE, ReplicatedLinear  # noqa: F401
from .mixtral_moe import FusedMoE  # noqa: F401
from .moe_align_block_size import moe_align_block_size  # noqa: F401
