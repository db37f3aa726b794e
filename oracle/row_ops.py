"""Oracle (test infrastructure): row reductions and dense GEMM on the CPU."""

from __future__ import annotations

import torch


def r16(x: torch.Tensor) -> torch.Tensor:
    """Round fp32 to bf16 (nearest even) and widen back."""
    return x.to(torch.bfloat16).to(torch.float32)


def matmul_ref(a: torch.Tensor, b: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``C = cast(sum_k f32(a) f32(b) + f32(bias))``: fp32 accumulate, bias added before the final
    cast (vexact/batch_invariant_ops/batch_invariant_ops.py:104-131)."""
    acc = a.to(torch.float32) @ b.to(torch.float32)
    if bias is not None:
        acc = acc + bias.to(torch.float32)
    return acc.to(a.dtype)


def mean_dim_ref(x: torch.Tensor, dim: int, keepdim: bool = False, dtype=None) -> torch.Tensor:
    """fp32 sum over ``dim`` divided by its length, stored in the working dtype
    (batch_invariant_ops.py:366-379, dtype rules :411-421)."""
    if dtype is None:
        dtype = torch.float32 if x.dtype in (torch.int8, torch.int16, torch.int32, torch.int64) else x.dtype
    x = x.to(dtype)
    n = x.shape[dim]
    return (x.to(torch.float32).sum(dim=dim, keepdim=keepdim) / n).to(dtype)


def rms_norm_ref(x: torch.Tensor, w: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """One rounding: ``cast(f32(x) * (1/sqrt(sum x^2 / n + eps)) * f32(w))``
    (batch_invariant_ops.py:653-669)."""
    xf = x.to(torch.float32)
    inv = 1.0 / torch.sqrt(xf.pow(2).sum(-1, keepdim=True) / x.shape[-1] + eps)
    return (xf * inv * w.to(torch.float32)).to(x.dtype)


def hf_rms_norm_ref(x: torch.Tensor, w: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """HuggingFace Qwen3 RMSNorm as it runs under the overrides: variance through the fp32 mean
    (batch_invariant_ops.py:619-622), ``x * rsqrt(var + eps)`` rounded to the input dtype, then
    multiplied by the weight in that dtype - two roundings."""
    xf = x.to(torch.float32)
    var = xf.pow(2).mean(-1, keepdim=True)
    t = (xf * torch.rsqrt(var + eps)).to(x.dtype)
    return w.to(x.dtype) * t


def log_softmax_ref(x: torch.Tensor) -> torch.Tensor:
    """``x - max - log(sum exp(x - max))`` over the last dim in fp32 (batch_invariant_ops.py:250-291)."""
    xf = x.to(torch.float32)
    m = xf.max(dim=-1, keepdim=True).values
    s = torch.exp(xf - m).sum(dim=-1, keepdim=True)
    return (xf - m - torch.log(s)).to(x.dtype)


def logprobs_ref(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """``log_softmax(logits)[label]`` in fp32: minus the cross-entropy the reference computes
    (vexact/batch_invariant_ops/standalone_logprobs.py:45-53)."""
    lp = log_softmax_ref(logits.to(torch.float32))
    return lp.gather(-1, labels.reshape(-1, 1).to(torch.int64)).squeeze(-1)
