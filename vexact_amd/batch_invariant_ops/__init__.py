"""Drop-in for ``vexact.batch_invariant_ops`` (export list of ``vexact/batch_invariant_ops/__init__.py:36-53``).

All four attention-interface names of the reference resolve to the one HIP implementation: the
FA3 / FA4 / flex / Triton back ends differ in kernels, not in interface.
"""

from .batch_invariant_ops import (
    AttentionBlockSize,
    batch_invariant_rms_norm,
    disable_batch_invariant_mode,
    enable_batch_invariant_mode,
    get_batch_invariant_attention_block_size,
    is_batch_invariant_mode_enabled,
    log_softmax,
    matmul_persistent,
    mean_dim,
    set_batch_invariant_mode,
    triton_bmm,
)
from .hip_invariant_attention import flash_attention_forward, flash_attn_varlen_func

flash_attention_forward_cute = flash_attention_forward
flex_attention_forward = flash_attention_forward
triton_flash_attention_forward = flash_attention_forward
triton_flash_attn_varlen_func = flash_attn_varlen_func

__version__ = "0.1.0"

__all__ = [
    "set_batch_invariant_mode",
    "is_batch_invariant_mode_enabled",
    "disable_batch_invariant_mode",
    "enable_batch_invariant_mode",
    "matmul_persistent",
    "log_softmax",
    "mean_dim",
    "get_batch_invariant_attention_block_size",
    "AttentionBlockSize",
    "flash_attention_forward",
    "flash_attention_forward_cute",
    "flex_attention_forward",
    "triton_flash_attn_varlen_func",
    "triton_flash_attention_forward",
    "triton_bmm",
    "batch_invariant_rms_norm",
]
