from .modeling_qwen3_moe import (
    Qwen3MoeExperts,
    apply_qwen3_moe_patches,
    invalidate_packed_experts,
    moe_block_forward,
    moe_block_init,
    remove_qwen3_moe_patches,
)

__all__ = ["Qwen3MoeExperts", "apply_qwen3_moe_patches", "remove_qwen3_moe_patches", "invalidate_packed_experts",
           "moe_block_forward", "moe_block_init"]
