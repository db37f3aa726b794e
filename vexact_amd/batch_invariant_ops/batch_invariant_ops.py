"""Batch-invariant aten overrides and public ops, backed by the HIP library.

Mirrors ``vexact/batch_invariant_ops/batch_invariant_ops.py`` of the reference:
``matmul_persistent`` (:158-228), ``log_softmax`` (:294-333), ``mean_dim`` (:384-473),
``triton_bmm`` (:567-606), ``batch_invariant_rms_norm`` (:728-730) and the mode switch
(:737-781). Same names, argument meaning and error behaviour; ``triton_bmm`` keeps its name
although no Triton is involved.
"""

from __future__ import annotations

import contextlib
import os
from collections import namedtuple

import torch

from .. import ops

__all__ = [
    "set_batch_invariant_mode",
    "is_batch_invariant_mode_enabled",
    "disable_batch_invariant_mode",
    "enable_batch_invariant_mode",
    "matmul_persistent",
    "log_softmax",
    "mean_dim",
    "triton_bmm",
    "batch_invariant_rms_norm",
    "get_batch_invariant_attention_block_size",
    "AttentionBlockSize",
]


def matmul_persistent(a: torch.Tensor, b: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``a @ b (+ bias)``; fp32 accumulation in ascending K, no split-K, output dtype = input dtype."""
    return ops.matmul(a, b, bias)


def log_softmax(input: torch.Tensor, dim: int = -1) -> torch.Tensor:
    """log_softmax along the last dimension (``ValueError`` for any other ``dim``)."""
    return ops.log_softmax(input, dim)


def mean_dim(
    input: torch.Tensor, dim: int, keepdim: bool = False, dtype: torch.dtype | None = None
) -> torch.Tensor:
    """Mean along one dimension with a fixed per-row reduction order."""
    assert input.is_cuda, "Input must be a CUDA tensor"
    return ops.mean_dim(input, dim, keepdim=keepdim, dtype=dtype)


def triton_bmm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Deterministic batched matmul ``(B, M, K) x (B, K, N) -> (B, M, N)``."""
    return ops.bmm(a, b)


def mm_batch_invariant(a, b):
    return matmul_persistent(a, b)


def addmm_batch_invariant(bias, a, b):
    # like the reference override, alpha/beta are not forwarded (they are 1 for nn.Linear)
    return matmul_persistent(a, b, bias=bias)


def bmm_batch_invariant(a, b):
    return triton_bmm(a, b)


def _log_softmax_batch_invariant(input, dim, _half_to_float):
    assert not _half_to_float, "not implemented"
    return log_softmax(input, dim=dim)


def mean_batch_invariant(input, dim, keepdim=False, dtype: torch.dtype | None = None):
    assert dtype is None or dtype == torch.float32, f"unsupported dtype: {dtype}"
    if len(dim) == 1:
        return mean_dim(input, dim[0], keepdim=keepdim)
    assert input.dtype in {torch.float16, torch.bfloat16, torch.float32}, "only float types supported for now"
    if len(dim) == 0:
        dim = list(range(input.ndim))
    n_elems = 1
    for d in dim:
        n_elems *= input.shape[d]
    return torch.sum(input, dim=dim, keepdim=keepdim, dtype=torch.float32).to(dtype or input.dtype) / n_elems


class BatchInvariantRMSNormFunction(torch.autograd.Function):
    """One-rounding RMSNorm (the reference's ``_rms_norm_kernel`` form) on the HIP kernels, forward and backward.
    The reference's backward is a chain of fp32 tensor operations (batch_invariant_ops.py:701-725); here
    ``ops.rms_norm_backward`` computes the same derivative, ``d_x = inv (d - h mean(d h))`` with ``h = x inv``,
    ``d = d_y w``, and ``d_w = sum d_y h``, in one kernel plus an ordered reduction. Rows it does not take (fp32,
    more than 8192 entries, a length that is not a multiple of 8) go through the tensor operations."""

    @staticmethod
    def forward(ctx, input, weight, eps):
        output = ops.rms_norm(input, weight, eps, hf_two_rounding=False)
        ctx.save_for_backward(input, weight)
        ctx.eps = eps
        return output

    @staticmethod
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        n = input.shape[-1]
        if input.dtype in (torch.bfloat16, torch.float16) and n % 8 == 0 and n <= 8192:
            d_x, d_w = ops.rms_norm_backward(input, weight, grad_output, ctx.eps, hf_two_rounding=False)
            return (d_x if ctx.needs_input_grad[0] else None), (d_w.to(weight.dtype) if ctx.needs_input_grad[1] else None), None
        x = input.float()
        inv_rms = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + ctx.eps)
        normed = x * inv_rms
        g = grad_output.float()
        grad_weight = (g * normed).reshape(-1, n).sum(0).to(weight.dtype)
        d = g * weight.float()
        grad_input = (inv_rms * (d - normed * (d * normed).mean(-1, keepdim=True))).to(input.dtype)
        return grad_input, grad_weight, None


def batch_invariant_rms_norm(input: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    return BatchInvariantRMSNormFunction.apply(input, weight, eps)


_batch_invariant_MODE = False
_batch_invariant_LIB = None


def is_batch_invariant_mode_enabled():
    return _batch_invariant_MODE


def _dispatch_key() -> str:
    acc = torch.accelerator.current_accelerator() if hasattr(torch, "accelerator") else None
    return getattr(acc, "type", "cpu").upper()  # "CUDA" on ROCm builds too


def enable_batch_invariant_mode():
    global _batch_invariant_MODE, _batch_invariant_LIB
    if _batch_invariant_MODE:
        return
    key = _dispatch_key()
    _batch_invariant_MODE = True
    _batch_invariant_LIB = torch.library.Library("aten", "IMPL")
    _batch_invariant_LIB.impl("aten::mm", mm_batch_invariant, key)
    _batch_invariant_LIB.impl("aten::addmm", addmm_batch_invariant, key)
    _batch_invariant_LIB.impl("aten::_log_softmax", _log_softmax_batch_invariant, key)
    _batch_invariant_LIB.impl("aten::mean.dim", mean_batch_invariant, key)

    os.environ.setdefault("CUBLAS_WORKSPACE_CONFIG", ":16:8")
    torch.backends.cuda.matmul.allow_bf16_reduced_precision_reduction = False
    torch.backends.cuda.matmul.allow_fp16_reduced_precision_reduction = False
    torch.use_deterministic_algorithms(True, warn_only=False)
    torch.backends.cudnn.deterministic = True


def disable_batch_invariant_mode():
    global _batch_invariant_MODE, _batch_invariant_LIB
    if _batch_invariant_LIB is not None:
        _batch_invariant_LIB._destroy()
    _batch_invariant_MODE = False
    _batch_invariant_LIB = None


@contextlib.contextmanager
def set_batch_invariant_mode(enabled: bool = True):
    """Switch the mode for the duration of the block and restore the previous state afterwards."""
    was_enabled = _batch_invariant_MODE
    if enabled:
        enable_batch_invariant_mode()
    else:
        disable_batch_invariant_mode()
    try:
        yield
    finally:
        if was_enabled:
            enable_batch_invariant_mode()
        else:
            disable_batch_invariant_mode()


AttentionBlockSize = namedtuple("AttentionBlockSize", ["block_m", "block_n"])


def get_batch_invariant_attention_block_size() -> AttentionBlockSize:
    return AttentionBlockSize(block_m=16, block_n=16)
