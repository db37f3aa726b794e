from .modeling_qwen3_moe import Qwen3MoeExperts, apply_qwen3_moe_patches, moe_block_forward, moe_block_init

__all__ = ["Qwen3MoeExperts", "apply_qwen3_moe_patches", "moe_block_forward", "moe_block_init"]
