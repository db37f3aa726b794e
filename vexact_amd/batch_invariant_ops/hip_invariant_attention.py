"""FlashAttention-compatible varlen interface and HuggingFace attention wrapper on the HIP kernels.

Mirrors ``vexact/batch_invariant_ops/triton_invariant_attention.py`` of the reference:
``flash_attn_varlen_func`` (:905-979), ``flash_attention_forward`` (:982-1088), the argument checks
of ``_PagedFlashAttentionVarlen.forward`` (:605-650) and the helpers at :13-44. The paged path raises
on backward like the reference (:694-697); the packed path has forward and backward
(``_NonpagedFlashAttentionVarlen``, :700-902).
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from .kv_cache_context import get_kv_cache_context, store_kvcache


def _require_cuda(name: str, tensor: torch.Tensor) -> None:
    if not tensor.is_cuda:
        raise ValueError(f"{name} must be a CUDA tensor")


def _require_cuda_int32(name: str, tensor: torch.Tensor) -> None:
    _require_cuda(name, tensor)
    if tensor.dtype != torch.int32:
        raise ValueError(f"{name} must have dtype torch.int32, got {tensor.dtype}")


def _check_common_args(dropout_p, softcap, window_size) -> None:
    if dropout_p != 0.0:
        raise NotImplementedError("triton flash_attn_varlen_func only supports dropout_p=0.0")
    if softcap is not None:
        raise NotImplementedError("triton flash_attn_varlen_func does not support softcap")
    if window_size is not None and window_size != (-1, -1):
        raise NotImplementedError("triton flash_attn_varlen_func does not support sliding-window attention")


def _default_softmax_scale(q: torch.Tensor, softmax_scale) -> float:
    if softmax_scale is None:
        return q.shape[-1] ** -0.5
    if isinstance(softmax_scale, torch.Tensor):
        raise ValueError("softmax_scale must be a Python float, not a tensor")
    return float(softmax_scale)


def _as_python_int(value, name: str) -> int:
    if isinstance(value, torch.Tensor):
        raise ValueError(f"{name} must be a Python int, not a tensor")
    return int(value)


class _PagedAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, seqused_k, page_table, softmax_scale, causal, max_seqlen_q):
        _require_cuda("q", q)
        _require_cuda("k", k)
        _require_cuda("v", v)
        _require_cuda_int32("page_table", page_table)
        _require_cuda_int32("cu_seqlens_q", cu_seqlens_q)
        _require_cuda_int32("seqused_k", seqused_k)
        if k.ndim != 4 or v.ndim != 4:
            raise ValueError("paged flash_attn_varlen_func expects k/v with shape (num_blocks, page_size, heads, dim)")
        if q.ndim != 3:
            raise ValueError("paged flash_attn_varlen_func expects q with shape (total_q, heads, dim)")
        if q.shape[-1] != k.shape[-1]:
            raise ValueError(f"q and k head_dim must match, got {q.shape[-1]} and {k.shape[-1]}")
        if q.shape[1] % k.shape[2] != 0:
            raise ValueError(f"query heads ({q.shape[1]}) must be divisible by KV heads ({k.shape[2]})")
        for name, t in (("cu_seqlens_q", cu_seqlens_q), ("seqused_k", seqused_k), ("page_table", page_table)):
            if t.device != q.device:
                raise ValueError(f"{name} must be on {q.device}, got {t.device}")
        if not causal:
            raise NotImplementedError("paged triton flash_attn_varlen_func only supports causal=True")
        if max(q.shape[-1], v.shape[-1]) > 256:
            raise ValueError(f"head_dim must be <= 256, got {q.shape[-1]}")
        if page_table.stride(-1) != 1:
            page_table = page_table.contiguous()
        return ops.paged_attention(
            q, k, v, cu_seqlens_q.contiguous(), seqused_k.contiguous(), page_table, softmax_scale, max_seqlen_q
        )

    @staticmethod
    def backward(ctx, do):
        raise NotImplementedError("paged triton flash_attn_varlen_func backward is not implemented")


class _PackedAttention(torch.autograd.Function):
    """Causal varlen attention on packed q/k/v with the HIP forward (log-sum-exp saved) and backward."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, cu_seqlens_k, softmax_scale, causal, max_seqlen_q, max_seqlen_k):
        if q.ndim != 3 or k.ndim != 3 or v.ndim != 3:
            raise ValueError("non-paged flash_attn_varlen_func expects q/k/v with shape (total_tokens, heads, head_dim)")
        if q.shape[-1] != k.shape[-1]:
            raise ValueError(f"q and k head_dim must match, got {q.shape[-1]} and {k.shape[-1]}")
        if k.shape[-2] != v.shape[-2]:
            raise ValueError(f"k/v must have the same number of KV heads, got {k.shape[-2]} and {v.shape[-2]}")
        if q.shape[-2] % k.shape[-2] != 0:
            raise ValueError(f"query heads ({q.shape[-2]}) must be divisible by KV heads ({k.shape[-2]})")
        if not causal:
            raise NotImplementedError("non-paged triton flash_attn_varlen_func only supports causal=True")
        q, k, v = (t if t.stride(-1) == 1 else t.contiguous() for t in (q, k, v))
        out, lse = ops.packed_attention(q, k, v, cu_seqlens_q, cu_seqlens_k, softmax_scale, True, max_seqlen_q,
                                        return_lse=True)
        ctx.save_for_backward(q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k)
        ctx.softmax_scale, ctx.max_seqlen_q, ctx.max_seqlen_k = softmax_scale, max_seqlen_q, max_seqlen_k
        return out

    @staticmethod
    def backward(ctx, do):
        q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k = ctx.saved_tensors
        if do.stride(-1) != 1:
            do = do.contiguous()
        dq, dk, dv = ops.packed_attention_backward(q, k, v, out, do, lse, cu_seqlens_q, cu_seqlens_k, ctx.softmax_scale,
                                                   ctx.max_seqlen_q, ctx.max_seqlen_k)
        return dq, dk, dv, None, None, None, None, None, None


def flash_attn_varlen_func(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: Optional[torch.Tensor] = None,
    max_seqlen_q: Optional[int] = None,
    max_seqlen_k: Optional[int] = None,
    dropout_p: float = 0.0,
    softmax_scale: Optional[float] = None,
    causal: bool = False,
    window_size: Optional[tuple[int, int]] = None,
    softcap: Optional[float] = None,
    alibi_slopes: Optional[torch.Tensor] = None,
    deterministic: bool = False,
    return_attn_probs: bool = False,
    block_table: Optional[torch.Tensor] = None,
    page_table: Optional[torch.Tensor] = None,
    seqused_k: Optional[torch.Tensor] = None,
    cache_seqlens: Optional[torch.Tensor] = None,
    **kwargs,
) -> tuple[torch.Tensor, None]:
    """``page_table`` / ``block_table`` are aliases. With one of them ``k``/``v`` are paged caches
    ``(blocks, page, Hkv, D)`` and ``seqused_k`` (or ``cache_seqlens``) holds the KV lengths; without,
    ``k``/``v`` are packed ``(total_k, Hkv, D)`` with ``cu_seqlens_k``. Returns ``(out, None)``."""
    del alibi_slopes, deterministic, return_attn_probs, kwargs
    _check_common_args(dropout_p, softcap, window_size)
    if page_table is not None and block_table is not None:
        raise ValueError("pass only one of page_table or block_table")
    scale = _default_softmax_scale(q, softmax_scale)
    table = page_table if page_table is not None else block_table
    if table is None:
        if cu_seqlens_q is None:
            raise ValueError("cu_seqlens_q is required when page_table/block_table is not provided")
        if cu_seqlens_k is None:
            raise ValueError("cu_seqlens_k is required when page_table/block_table is not provided")
        if max_seqlen_k is None:
            raise ValueError("max_seqlen_k is required when page_table/block_table is not provided")
        if max_seqlen_q is None:
            raise ValueError("max_seqlen_q is required when page_table/block_table is not provided")
        _require_cuda("q", q)
        _require_cuda_int32("cu_seqlens_q", cu_seqlens_q)
        _require_cuda_int32("cu_seqlens_k", cu_seqlens_k)
        if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
            out = _PackedAttention.apply(
                q, k, v, cu_seqlens_q.contiguous(), cu_seqlens_k.contiguous(), scale, bool(causal),
                _as_python_int(max_seqlen_q, "max_seqlen_q"), _as_python_int(max_seqlen_k, "max_seqlen_k"),
            )
            return out, None
        _as_python_int(max_seqlen_k, "max_seqlen_k")
        out = ops.packed_attention(
            q, k, v, cu_seqlens_q.contiguous(), cu_seqlens_k.contiguous(), scale, bool(causal),
            _as_python_int(max_seqlen_q, "max_seqlen_q"),
        )
        return out, None

    lens = seqused_k if seqused_k is not None else cache_seqlens
    if lens is None:
        raise ValueError("seqused_k or cache_seqlens is required when page_table/block_table is provided")
    if max_seqlen_q is None:
        max_seqlen_q = 0
    out = _PagedAttention.apply(
        q, k, v, cu_seqlens_q, lens, table, scale, causal, _as_python_int(max_seqlen_q, "max_seqlen_q")
    )
    return out, None


def flash_attention_forward(
    module: nn.Module,
    query: torch.Tensor,
    key: Optional[torch.Tensor],
    value: Optional[torch.Tensor],
    attention_mask: Optional[torch.Tensor],
    scaling: float,
    dropout: float = 0.0,
    **kwargs,
) -> tuple[torch.Tensor, None]:
    """HuggingFace ``ALL_ATTENTION_FUNCTIONS`` entry: ``query [B,Hq,Q,D]``, ``key/value [B,Hkv,K,D]``.
    With a paged context it stores the new K/V at ``slot_mapping`` and attends over the cache,
    returning ``(out [T,Hq,Dv], None)``."""
    ctx = get_kv_cache_context()
    query = query.transpose(1, 2).contiguous()
    if key is not None:
        key = key.transpose(1, 2).contiguous()
    if value is not None:
        value = value.transpose(1, 2).contiguous()
    _, _, num_heads, head_dim = query.shape
    layer_idx = _as_python_int(
        kwargs.get("layer_idx") if "layer_idx" in kwargs else getattr(module, "layer_idx", 0), "layer_idx"
    )

    if ctx is None:
        if key is None or value is None:
            raise ValueError("key and value are required for non-paged triton attention")
        batch_size, q_len = query.shape[:2]

        def pick(*names):
            for n in names:
                if kwargs.get(n) is not None:
                    return kwargs[n]
            return None

        cu_q = pick("cu_seq_lens_q", "cu_seqlens_q", "cu_seq_lens", "cu_seqlens")
        cu_k = pick("cu_seq_lens_k", "cu_seqlens_k", "cu_seq_lens", "cu_seqlens")
        max_q = pick("max_length_q", "max_seqlen_q", "max_seqlen")
        max_k = pick("max_length_k", "max_seqlen_k", "max_seqlen")
        if cu_q is None:
            raise ValueError("cu_seq_lens_q/cu_seqlens_q is required for non-paged triton-invariant attention")
        if cu_k is None:
            raise ValueError("cu_seq_lens_k/cu_seqlens_k is required for non-paged triton-invariant attention")
        if max_q is None:
            raise ValueError("max_length_q/max_seqlen_q is required for non-paged triton-invariant attention")
        if max_k is None:
            raise ValueError("max_length_k/max_seqlen_k is required for non-paged triton-invariant attention")
        out, _ = flash_attn_varlen_func(
            query.reshape(-1, num_heads, head_dim),
            key.reshape(-1, key.shape[2], key.shape[-1]),
            value.reshape(-1, value.shape[2], value.shape[-1]),
            cu_seqlens_q=cu_q, cu_seqlens_k=cu_k, max_seqlen_q=max_q, max_seqlen_k=max_k,
            dropout_p=dropout, softmax_scale=scaling,
            causal=kwargs.get("is_causal", getattr(module, "is_causal", True)),
        )
        return out.reshape(batch_size, q_len, num_heads, -1), None

    if ctx.is_paged_attn:
        k_blocks = ctx.key_cache[layer_idx]
        v_blocks = ctx.value_cache[layer_idx]
        if key is not None and value is not None:
            hkv = key.shape[2]
            store_kvcache(
                key.reshape(-1, hkv, head_dim), value.reshape(-1, hkv, value.shape[-1]), k_blocks, v_blocks,
                ctx.slot_mapping,
            )
        return flash_attn_varlen_func(
            query.reshape(-1, num_heads, head_dim), k_blocks, v_blocks,
            cu_seqlens_q=ctx.query_start_loc, cu_seqlens_k=None, max_seqlen_q=ctx.max_seqlen_q, max_seqlen_k=None,
            seqused_k=ctx.context_lens, page_table=ctx.block_tables, dropout_p=dropout, softmax_scale=scaling,
            causal=True,
        )

    if key is None or value is None:
        raise ValueError("key and value are required for non-paged triton attention")
    return flash_attn_varlen_func(
        query.reshape(-1, num_heads, head_dim),
        key.reshape(-1, key.shape[2], key.shape[-1]),
        value.reshape(-1, value.shape[2], value.shape[-1]),
        cu_seqlens_q=ctx.query_start_loc, cu_seqlens_k=ctx.query_start_loc,
        max_seqlen_q=ctx.max_seqlen_q, max_seqlen_k=ctx.max_seqlen_q,
        dropout_p=dropout, softmax_scale=scaling, causal=True,
    )


__all__ = ["flash_attn_varlen_func", "flash_attention_forward"]
