"""Thread-local paged-KV context, block allocator, cache tensors and the cache scatter.

Mirrors ``vexact/batch_invariant_ops/kv_cache_context.py`` of the reference: ``KVCacheContext``
(:48-104), ``set/get/has_kv_cache_context`` (:107-138), ``KVCacheManager`` (:141-217),
``KVCacheStore`` (:220-253) and ``store_kvcache`` (:294-314, HIP kernel here).
"""

from __future__ import annotations

import ctypes
import threading
from dataclasses import dataclass
from typing import Iterable, Optional

import torch

from .. import _lib, ops

_context_storage = threading.local()


@dataclass(frozen=True)
class KVCacheInfo:
    layer_idxs: Iterable[int]
    num_kv_heads: int
    head_dim: int
    page_size: int
    max_blocks: int
    device: torch.device
    dtype: torch.dtype = torch.bfloat16


@dataclass
class KVCacheContext:
    """What the attention wrapper needs for one forward pass.

    ``block_tables [B, max_blocks]`` int32 (-1 padded), ``slot_mapping [T]`` int32 (-1 = do not
    store), ``context_lens [B]`` int32 (past + new tokens), ``query_start_loc [B+1]`` int32,
    ``max_seqlen_q`` host int.
    """

    is_paged_attn: bool = False
    key_cache: Optional[dict] = None
    value_cache: Optional[dict] = None
    block_tables: Optional[torch.Tensor] = None
    slot_mapping: Optional[torch.Tensor] = None
    context_lens: Optional[torch.Tensor] = None
    query_start_loc: Optional[torch.Tensor] = None
    max_seqlen_q: Optional[int] = None

    def __post_init__(self):
        if self.is_paged_attn:
            assert self.key_cache is not None, "key_cache required for paged attention"
            assert self.value_cache is not None, "value_cache required for paged attention"
            assert self.block_tables is not None, "block_tables required for paged attention"
            assert self.context_lens is not None, "context_lens required for paged attention"
        else:
            assert self.query_start_loc is not None, "query_start_loc required for packed attention"
            assert self.context_lens is not None, "context_lens required for packed attention"


def set_kv_cache_context(
    is_paged_attn: bool = False,
    key_cache=None,
    value_cache=None,
    block_tables: Optional[torch.Tensor] = None,
    context_lens: Optional[torch.Tensor] = None,
    slot_mapping: Optional[torch.Tensor] = None,
    query_start_loc: Optional[torch.Tensor] = None,
    max_seqlen_q: Optional[int] = None,
):
    _context_storage.kv_cache_context = KVCacheContext(
        is_paged_attn=is_paged_attn,
        key_cache=key_cache,
        value_cache=value_cache,
        block_tables=block_tables,
        context_lens=context_lens,
        slot_mapping=slot_mapping,
        query_start_loc=query_start_loc,
        max_seqlen_q=max_seqlen_q,
    )


def get_kv_cache_context() -> Optional[KVCacheContext]:
    return getattr(_context_storage, "kv_cache_context", None)


def has_kv_cache_context() -> bool:
    return hasattr(_context_storage, "kv_cache_context")


def clear_kv_cache_context() -> None:
    if hasattr(_context_storage, "kv_cache_context"):
        del _context_storage.kv_cache_context


class KVCacheManager:
    """Block allocator: always hands out the lowest free block id, ``None`` when out of blocks.

    Same observable behaviour as the reference allocator (kv_cache_context.py:141-217); the free
    list is a native min-heap (``vx_kv_allocator_*``), so an allocation costs O(log n) per block
    instead of a scan of the free set. Not thread-safe, like the reference's.
    """

    def __init__(self, cache_config):
        self.cache_config = cache_config
        self._lib = _lib.load()
        self._num_blocks = int(cache_config.max_cache_blocks)
        self._h = self._lib.vx_kv_allocator_create(self._num_blocks)
        if not self._h:
            raise ValueError(f"cannot create a block allocator for {cache_config.max_cache_blocks} blocks")
        self._out = (ctypes.c_int32 * max(1, self._num_blocks))()

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                self._lib.vx_kv_allocator_destroy(h)
            except Exception:  # interpreter shutdown: the library may already be gone
                pass

    def _num_blocks_needed(self, num_tokens: int) -> int:
        return (num_tokens + self.cache_config.page_size - 1) // self.cache_config.page_size

    def allocate_blocks(self, total_tokens: int, num_current_blocks: int = 0):
        delta = self._num_blocks_needed(total_tokens) - num_current_blocks
        if delta <= 0:
            return []
        if delta > self._num_blocks:
            return None
        n = self._lib.vx_kv_allocator_allocate(self._h, int(delta), 0, 1, self._out, self._num_blocks)
        return None if n < 0 else self._out[:n]

    def num_free_blocks(self) -> int:
        return int(self._lib.vx_kv_allocator_num_free(self._h))

    def num_allocated_blocks(self) -> int:
        return self._num_blocks - self.num_free_blocks()

    def free_blocks(self, block_ids):
        ids = [int(b) for b in block_ids if -(2 ** 31) <= int(b) < 2 ** 31]
        if ids:
            self._lib.vx_kv_allocator_free(self._h, (ctypes.c_int32 * len(ids))(*ids), len(ids))


def _kv_head_dims(hf_config) -> tuple[int, int]:
    """(key head size, value head size): models with separate sizes (multi-head latent attention) name them
    ``qk_head_dim`` / ``v_head_dim``; the others have one ``head_dim`` or ``hidden_size / heads``."""
    base = getattr(hf_config, "head_dim", None) or hf_config.hidden_size // hf_config.num_attention_heads
    dk = getattr(hf_config, "qk_head_dim", base)
    return dk, getattr(hf_config, "v_head_dim", dk)


class KVCacheStore:
    """Paged key / value memory of a model: ``key_cache[layer]`` and ``value_cache[layer]`` are
    ``[max_cache_blocks, page_size, Hkv, D]`` tensors, zero initialised (reference: kv_cache_context.py:220-253).
    All layers of a kind live in ONE allocation (a ``[layers, blocks, page, Hkv, D]`` slab): two large
    allocations for the whole pool instead of two per layer, and the per-layer tensors are views of it."""

    def __init__(self, hf_config, cache_config, device: torch.device, head_major: bool = False):
        """``head_major`` (not in the reference): the memory is ``[layers, blocks, Hkv, page, D]`` and the per-layer
        tensors are its ``[blocks, page, Hkv, D]`` views, so a kv head's page is one contiguous piece; ``store_kvcache``
        and the attention wrappers take the views as they are, decode attention streams them about 15 % faster.
        The views are not contiguous: code that flattens a cache tensor with ``.view(-1, ...)`` needs the default."""
        self.hf_config, self.cache_config, self.device = hf_config, cache_config, device
        self.head_major = head_major
        self.page_size, self.max_blocks = cache_config.page_size, cache_config.max_cache_blocks
        dtype = getattr(hf_config, "dtype", None) or getattr(hf_config, "torch_dtype", None) or torch.bfloat16
        if isinstance(dtype, str):  # configs read from JSON carry the name
            dtype = getattr(torch, dtype.replace("torch.", ""))
        layers, heads = hf_config.num_hidden_layers, hf_config.num_key_value_heads
        if head_major:
            slabs = [torch.zeros((layers, self.max_blocks, heads, self.page_size, d), device=device, dtype=dtype).permute(0, 1, 3, 2, 4)
                     for d in _kv_head_dims(hf_config)]
        else:
            slabs = [torch.zeros((layers, self.max_blocks, self.page_size, heads, d), device=device, dtype=dtype)
                     for d in _kv_head_dims(hf_config)]
        self.key_cache: dict[int, torch.Tensor] = dict(enumerate(slabs[0].unbind(0)))
        self.value_cache: dict[int, torch.Tensor] = dict(enumerate(slabs[1].unbind(0)))


def store_kvcache(
    key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor
):
    """``cache.view(-1, H*D)[slot] = src`` for every token whose slot is not -1 (K and V may differ in D)."""
    ops.store_kvcache(key, value, k_cache, v_cache, slot_mapping)
