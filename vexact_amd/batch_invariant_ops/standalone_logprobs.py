"""Per-token log-probabilities; mirrors ``logprobs_from_logits_flash_attn`` of
``vexact/batch_invariant_ops/standalone_logprobs.py:28-55`` (which returns minus the cross-entropy
of flash-attn's Triton kernel: ``logits[i, label] - logsumexp(logits[i])`` in fp32, with that kernel's
backward and its ``inplace_backward`` option)."""

from __future__ import annotations

import torch

from .. import ops


class _LogprobsFunction(torch.autograd.Function):
    """Forward: the rollout's kernel (``vx_logprobs``), so a trainer scores tokens with the rollout's bits.
    Backward: ``d_logits = d_out (onehot(label) - softmax(logits))``, one kernel, optionally into the logits."""

    @staticmethod
    def forward(ctx, logits, labels, inplace_backward):
        flat = logits.reshape(-1, logits.shape[-1])
        out = ops.logprobs(flat, labels.reshape(-1))
        ctx.save_for_backward(flat, labels.reshape(-1), out)
        ctx.inplace, ctx.shape = bool(inplace_backward), logits.shape
        return out.reshape(labels.shape)

    @staticmethod
    def backward(ctx, d_out):
        flat, labels, out = ctx.saved_tensors
        x = flat if flat.stride(-1) == 1 else flat.contiguous()
        d = ops.logprobs_backward(x, labels, out, d_out.reshape(-1), inplace=ctx.inplace and x is flat)
        return d.reshape(ctx.shape), None, None


def logprobs_from_logits_flash_attn(
    logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = False
) -> torch.Tensor:
    if torch.is_grad_enabled() and logits.requires_grad:
        return _LogprobsFunction.apply(logits, labels, inplace_backward)
    shape = labels.shape
    out = ops.logprobs(logits.reshape(-1, logits.shape[-1]), labels.reshape(-1))
    return out.reshape(shape)
