from .modeling_qwen3_moe import (
    Qwen3MoeExperts,
    apply_qwen3_moe_patches,
    fuse_qkv_weights,
    invalidate_packed_experts,
    moe_block_forward,
    moe_block_init,
    remove_qwen3_moe_patches,
    unfuse_qkv_weights,
)

__all__ = ["Qwen3MoeExperts", "apply_qwen3_moe_patches", "remove_qwen3_moe_patches", "invalidate_packed_experts",
           "moe_block_forward", "moe_block_init", "fuse_qkv_weights", "unfuse_qkv_weights"]
