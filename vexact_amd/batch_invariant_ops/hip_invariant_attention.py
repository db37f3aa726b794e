"""FlashAttention-compatible varlen interface and HuggingFace attention wrapper on the HIP kernels.

Drop-in for ``vexact/batch_invariant_ops/triton_invariant_attention.py`` of the reference: the same two
public callables with the same signatures, return values and error messages
(``flash_attn_varlen_func`` :905-979, ``flash_attention_forward`` :982-1088; argument rules of the paged
and packed autograd functions :605-650, :700-740). The paged path raises on backward like the reference
(:694-697); the packed path has forward and backward.

The kernels take token and head strides, so the wrapper hands them views of HuggingFace's
``[batch, heads, tokens, dim]`` tensors instead of transposed copies; a copy is made only for a layout the
kernels cannot address (a head dimension that is not contiguous, strides that break 16-byte alignment).
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from .kv_cache_context import get_kv_cache_context

_WHO = "triton flash_attn_varlen_func"  # the name the reference's messages carry


# ----------------------------------------------------------------------------- argument rules
def _on_gpu(**tensors) -> None:
    for name, t in tensors.items():
        if not t.is_cuda:
            raise ValueError(f"{name} must be a CUDA tensor")


def _int32_on_gpu(**tensors) -> None:
    _on_gpu(**tensors)
    for name, t in tensors.items():
        if t.dtype != torch.int32:
            raise ValueError(f"{name} must have dtype torch.int32, got {t.dtype}")


def _host_int(name: str, value) -> int:
    if torch.is_tensor(value):
        raise ValueError(f"{name} must be a Python int, not a tensor")
    return int(value)


def _head_rules(q, k, v, heads_axis: int) -> None:
    """Shape rules shared by the paged and the packed form (``heads_axis`` of k / v)."""
    if q.shape[-1] != k.shape[-1]:
        raise ValueError(f"q and k head_dim must match, got {q.shape[-1]} and {k.shape[-1]}")
    if k.shape[heads_axis] != v.shape[heads_axis]:
        raise ValueError(f"k/v must have the same number of KV heads, got {k.shape[heads_axis]} and {v.shape[heads_axis]}")
    if q.shape[-2] % k.shape[heads_axis] != 0:
        raise ValueError(f"query heads ({q.shape[-2]}) must be divisible by KV heads ({k.shape[heads_axis]})")


def _addressable(t: torch.Tensor) -> torch.Tensor:
    """``[tokens, heads, dim]`` as the kernels read it fastest: unit stride in ``dim`` (required) and 16-byte
    aligned rows. A view whose rows a copy would align is copied; a head size that is not a multiple of 8 elements
    cannot be aligned and goes to the kernels as it is (they then access it element by element)."""
    if t.stride(-1) != 1:
        return t.contiguous()
    aligned = t.stride(0) % 8 == 0 and t.stride(1) % 8 == 0 and t.data_ptr() % 16 == 0
    return t if aligned or t.shape[-1] % 8 != 0 else t.contiguous()


# ----------------------------------------------------------------------------- autograd functions
class _PagedAttention(torch.autograd.Function):
    """Causal attention of packed queries over a paged cache; forward only."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, seqused_k, page_table, softmax_scale, causal, max_seqlen_q):
        _on_gpu(q=q, k=k, v=v)
        _int32_on_gpu(page_table=page_table, cu_seqlens_q=cu_seqlens_q, seqused_k=seqused_k)
        if k.ndim != 4 or v.ndim != 4:
            raise ValueError("paged flash_attn_varlen_func expects k/v with shape (num_blocks, page_size, heads, dim)")
        if q.ndim != 3:
            raise ValueError("paged flash_attn_varlen_func expects q with shape (total_q, heads, dim)")
        _head_rules(q, k, v, heads_axis=2)
        for name, t in (("cu_seqlens_q", cu_seqlens_q), ("seqused_k", seqused_k), ("page_table", page_table)):
            if t.device != q.device:
                raise ValueError(f"{name} must be on {q.device}, got {t.device}")
        if not causal:
            raise NotImplementedError(f"paged {_WHO} only supports causal=True")
        widest = max(q.shape[-1], v.shape[-1])
        if widest > 256:
            raise ValueError(f"head_dim must be <= 256, got {widest}")
        table = page_table if page_table.stride(-1) == 1 else page_table.contiguous()
        return ops.paged_attention(_addressable(q), k, v, cu_seqlens_q.contiguous(), seqused_k.contiguous(), table,
                                   softmax_scale, max_seqlen_q)

    @staticmethod
    def backward(ctx, do):
        raise NotImplementedError(f"paged {_WHO} backward is not implemented")


class _PackedAttention(torch.autograd.Function):
    """Causal varlen attention on packed q/k/v with the HIP forward (log-sum-exp saved) and backward."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, cu_seqlens_k, softmax_scale, max_seqlen_q, max_seqlen_k):
        q, k, v = _addressable(q), _addressable(k), _addressable(v)
        out, lse = ops.packed_attention(q, k, v, cu_seqlens_q, cu_seqlens_k, softmax_scale, True, max_seqlen_q,
                                        return_lse=True)
        ctx.save_for_backward(q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k)
        ctx.call = (softmax_scale, max_seqlen_q, max_seqlen_k)
        return out

    @staticmethod
    def backward(ctx, do):
        q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k = ctx.saved_tensors
        scale, max_q, max_k = ctx.call
        grads = ops.packed_attention_backward(q, k, v, out, _addressable(do), lse, cu_seqlens_q, cu_seqlens_k, scale,
                                              max_q, max_k)
        return (*grads, None, None, None, None, None)


def _packed(q, k, v, cu_seqlens_q, cu_seqlens_k, scale, causal, max_seqlen_q, max_seqlen_k):
    missing = {"cu_seqlens_q": cu_seqlens_q, "cu_seqlens_k": cu_seqlens_k, "max_seqlen_k": max_seqlen_k,
               "max_seqlen_q": max_seqlen_q}
    for name, value in missing.items():
        if value is None:
            raise ValueError(f"{name} is required when page_table/block_table is not provided")
    _on_gpu(q=q)
    _int32_on_gpu(cu_seqlens_q=cu_seqlens_q, cu_seqlens_k=cu_seqlens_k)
    if q.ndim != 3 or k.ndim != 3 or v.ndim != 3:
        raise ValueError("non-paged flash_attn_varlen_func expects q/k/v with shape (total_tokens, heads, head_dim)")
    _head_rules(q, k, v, heads_axis=-2)
    max_q, max_k = _host_int("max_seqlen_q", max_seqlen_q), _host_int("max_seqlen_k", max_seqlen_k)
    cu_q, cu_k = cu_seqlens_q.contiguous(), cu_seqlens_k.contiguous()
    if torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v)):
        if not causal:  # the reference has no non-causal form at all; here the forward kernel has one, the backward not
            raise NotImplementedError(f"non-paged {_WHO} only supports causal=True")
        return _PackedAttention.apply(q, k, v, cu_q, cu_k, scale, max_q, max_k)
    return ops.packed_attention(_addressable(q), _addressable(k), _addressable(v), cu_q, cu_k, scale, causal, max_q)


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
    unsupported = ((dropout_p != 0.0, "only supports dropout_p=0.0"),
                   (softcap is not None, "does not support softcap"),
                   (window_size is not None and window_size != (-1, -1), "does not support sliding-window attention"))
    for hit, what in unsupported:
        if hit:
            raise NotImplementedError(f"{_WHO} {what}")
    if page_table is not None and block_table is not None:
        raise ValueError("pass only one of page_table or block_table")
    if torch.is_tensor(softmax_scale):
        raise ValueError("softmax_scale must be a Python float, not a tensor")
    scale = q.shape[-1] ** -0.5 if softmax_scale is None else float(softmax_scale)

    table = block_table if page_table is None else page_table
    if table is None:
        return _packed(q, k, v, cu_seqlens_q, cu_seqlens_k, scale, bool(causal), max_seqlen_q, max_seqlen_k), None
    kv_lens = cache_seqlens if seqused_k is None else seqused_k
    if kv_lens is None:
        raise ValueError("seqused_k or cache_seqlens is required when page_table/block_table is provided")
    max_q = 0 if max_seqlen_q is None else _host_int("max_seqlen_q", max_seqlen_q)
    return _PagedAttention.apply(q, k, v, cu_seqlens_q, kv_lens, table, scale, causal, max_q), None


# ----------------------------------------------------------------------------- HuggingFace interface
def _token_rows(x: torch.Tensor) -> torch.Tensor:
    """HuggingFace's ``[batch, heads, tokens, dim]`` as ``[batch * tokens, heads, dim]`` without moving data
    when the batch is 1 (the packed case): a strided view the kernels read directly."""
    if x.shape[0] == 1:
        return x[0].transpose(0, 1)
    x = x.transpose(1, 2)
    return x.reshape(-1, x.shape[2], x.shape[3])


def _first_given(kwargs: dict, *names):
    return next((kwargs[n] for n in names if kwargs.get(n) is not None), None)


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
    returning ``(out [T,Hq,Dv], None)``; with a packed context or none, over the given K/V."""
    kv_ctx = get_kv_cache_context()
    batch, _, q_len, _ = query.shape
    layer_idx = _host_int("layer_idx", kwargs["layer_idx"] if "layer_idx" in kwargs else getattr(module, "layer_idx", 0))
    q = _token_rows(query)
    have_kv = key is not None and value is not None
    paged = kv_ctx is not None and kv_ctx.is_paged_attn
    if not paged and not have_kv:
        raise ValueError("key and value are required for non-paged triton attention")
    k, v = (_token_rows(key), _token_rows(value)) if have_kv else (None, None)

    if paged:
        k_blocks, v_blocks = kv_ctx.key_cache[layer_idx], kv_ctx.value_cache[layer_idx]
        if have_kv:  # this step's keys and values go into the cache first
            rows = [t if t.stride(-1) == 1 and t.stride(1) == t.shape[-1] else t.contiguous() for t in (k, v)]
            ops.store_kvcache(rows[0], rows[1], k_blocks, v_blocks, kv_ctx.slot_mapping)
        return flash_attn_varlen_func(
            q, k_blocks, v_blocks, cu_seqlens_q=kv_ctx.query_start_loc, max_seqlen_q=kv_ctx.max_seqlen_q,
            seqused_k=kv_ctx.context_lens, page_table=kv_ctx.block_tables, dropout_p=dropout, softmax_scale=scaling,
            causal=True)

    if kv_ctx is not None:  # packed context: queries and keys share the sequence boundaries
        return flash_attn_varlen_func(
            q, k, v, cu_seqlens_q=kv_ctx.query_start_loc, cu_seqlens_k=kv_ctx.query_start_loc,
            max_seqlen_q=kv_ctx.max_seqlen_q, max_seqlen_k=kv_ctx.max_seqlen_q, dropout_p=dropout,
            softmax_scale=scaling, causal=True)

    # no context: sequence boundaries come with the call, under any of the names HuggingFace models use
    bounds = {
        "cu_seq_lens_q/cu_seqlens_q": _first_given(kwargs, "cu_seq_lens_q", "cu_seqlens_q", "cu_seq_lens", "cu_seqlens"),
        "cu_seq_lens_k/cu_seqlens_k": _first_given(kwargs, "cu_seq_lens_k", "cu_seqlens_k", "cu_seq_lens", "cu_seqlens"),
        "max_length_q/max_seqlen_q": _first_given(kwargs, "max_length_q", "max_seqlen_q", "max_seqlen"),
        "max_length_k/max_seqlen_k": _first_given(kwargs, "max_length_k", "max_seqlen_k", "max_seqlen"),
    }
    for name, value_ in bounds.items():
        if value_ is None:
            raise ValueError(f"{name} is required for non-paged triton-invariant attention")
    cu_q, cu_k, max_q, max_k = bounds.values()
    out, _ = flash_attn_varlen_func(
        q, k, v, cu_seqlens_q=cu_q, cu_seqlens_k=cu_k, max_seqlen_q=max_q, max_seqlen_k=max_k, dropout_p=dropout,
        softmax_scale=scaling, causal=kwargs.get("is_causal", getattr(module, "is_causal", True)))
    return out.reshape(batch, q_len, q.shape[1], -1), None


__all__ = ["flash_attn_varlen_func", "flash_attention_forward"]
