"""MoE routing helpers on the HIP kernels; mirrors ``expert_histogram`` (:52-81), ``moe_gather``
(:131-161) and ``moe_scatter`` (:304-335) of
``vexact/batch_invariant_ops/group_gemm/kernel/moe.py``."""

from __future__ import annotations

import torch

from .... import ops


def expert_histogram(input: torch.Tensor, num_bins: int) -> torch.Tensor:
    """``out[e]`` = number of entries of ``input`` equal to ``e`` (int32, exact)."""
    return ops.expert_histogram(input, num_bins)


def moe_scatter(x: torch.Tensor, index: torch.Tensor, out_dtype=None) -> torch.Tensor:
    """``out[index[t, i]] = x[t]`` for every slot ``i``."""
    return ops.moe_scatter(x, index, out_dtype)


def moe_gather(x: torch.Tensor, index: torch.Tensor, out_dtype=None) -> torch.Tensor:
    """``y[t] = sum_i x[index[t, i]]`` summed in fp32 in slot order, then rounded."""
    return ops.moe_gather(x, index, out_dtype)
