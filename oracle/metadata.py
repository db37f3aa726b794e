"""Oracle (test infrastructure): integer metadata of one inference step."""

from __future__ import annotations

import numpy as np


def prepare_gen_ctx_ref(requests, page_size: int, max_blocks_per_req: int):
    """``requests``: list of dicts with ``num_computed_tokens`` (after this step), ``tokens_this_step``
    and ``block_ids``. Builds ``slot_mapping`` (-1 default, ``block_id * page + offset``),
    ``context_lens``, ``block_tables`` (-1 padded), ``query_start_loc``, ``max_seqlen_q`` and the
    positions, token by token (vexact/inferencer/inferencer.py:193-291)."""
    total = sum(r["tokens_this_step"] for r in requests)
    slot_mapping = np.full((total,), -1, dtype=np.int32)
    positions = np.zeros((total,), dtype=np.int64)
    i = 0
    for r in requests:
        start = r["num_computed_tokens"] - r["tokens_this_step"]
        assert start >= 0
        for pos in range(start, start + r["tokens_this_step"]):
            slot_mapping[i] = r["block_ids"][pos // page_size] * page_size + pos % page_size
            positions[i] = pos
            i += 1
    context_lens = np.array([r["num_computed_tokens"] for r in requests], dtype=np.int32)
    block_tables = np.full((len(requests), max_blocks_per_req), -1, dtype=np.int32)
    for s, r in enumerate(requests):
        for j, b in enumerate(r["block_ids"]):
            block_tables[s, j] = b
    qsl = np.zeros((len(requests) + 1,), dtype=np.int32)
    for s, r in enumerate(requests):
        qsl[s + 1] = qsl[s] + r["tokens_this_step"]
    max_q = max((r["tokens_this_step"] for r in requests), default=0)
    return {
        "slot_mapping": slot_mapping,
        "context_lens": context_lens,
        "block_tables": block_tables,
        "query_start_loc": qsl,
        "max_seqlen_q": max_q,
        "positions": positions,
    }


def pad_for_graph_ref(ctx, capture_tokens: int, graph_num_seqs: int):
    """Static-buffer padding for a captured bucket (vexact/inferencer/inferencer.py:306-324): pad
    tokens get slot -1 and position 0; pad sequences get ``query_start_loc = total_tokens``,
    ``context_len = 0`` and an all-zero block-table row."""
    T = ctx["slot_mapping"].shape[0]
    B = ctx["context_lens"].shape[0]
    assert T <= capture_tokens and B <= graph_num_seqs
    slot = np.full((capture_tokens,), -1, np.int32)
    slot[:T] = ctx["slot_mapping"]
    pos = np.zeros((capture_tokens,), np.int64)
    pos[:T] = ctx["positions"]
    lens = np.zeros((graph_num_seqs,), np.int32)
    lens[:B] = ctx["context_lens"]
    bt = np.full((graph_num_seqs, ctx["block_tables"].shape[1]), -1, np.int32)
    bt[:B] = ctx["block_tables"]
    bt[B:] = 0
    qsl = np.zeros((graph_num_seqs + 1,), np.int32)
    qsl[: B + 1] = ctx["query_start_loc"]
    qsl[B + 1 :] = T
    return {"slot_mapping": slot, "positions": pos, "context_lens": lens, "block_tables": bt,
            "query_start_loc": qsl, "max_seqlen_q": ctx["max_seqlen_q"]}


class BlockAllocatorRef:
    """Scan-based restatement of the block allocator (vexact/batch_invariant_ops/kv_cache_context.py:
    141-217): a set of free ids, ``min`` of it per allocated block, frees only ids it handed out."""

    def __init__(self, num_blocks: int, page_size: int):
        self.page_size = page_size
        self.allocated = set()
        self.free = set(range(num_blocks))

    def allocate(self, total_tokens: int, num_current_blocks: int = 0):
        delta = (total_tokens + self.page_size - 1) // self.page_size - num_current_blocks
        if delta <= 0:
            return []
        if len(self.free) < delta:
            return None
        out = []
        for _ in range(delta):
            b = min(self.free)
            self.free.remove(b)
            self.allocated.add(b)
            out.append(b)
        return out

    def release(self, block_ids):
        for b in block_ids:
            if b in self.allocated:
                self.allocated.remove(b)
                self.free.add(b)
