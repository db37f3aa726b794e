"""Per-token log-probabilities; mirrors ``logprobs_from_logits_flash_attn`` of
``vexact/batch_invariant_ops/standalone_logprobs.py:28-55`` (which returns minus the cross-entropy
of flash-attn's Triton kernel: ``logits[i, label] - logsumexp(logits[i])`` in fp32)."""

from __future__ import annotations

import torch

from .. import ops


def logprobs_from_logits_flash_attn(
    logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = False
) -> torch.Tensor:
    del inplace_backward  # forward only
    if logits.requires_grad:
        raise NotImplementedError("logprobs_from_logits_flash_attn is forward-only in this build")
    shape = labels.shape
    out = ops.logprobs(logits.reshape(-1, logits.shape[-1]), labels.reshape(-1))
    return out.reshape(shape)
