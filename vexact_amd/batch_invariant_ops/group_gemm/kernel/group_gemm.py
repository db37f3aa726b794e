"""Grouped GEMM with shared N, K on the HIP kernels; mirrors ``group_gemm_same_nk`` of
``vexact/batch_invariant_ops/group_gemm/kernel/group_gemm.py:156-237`` (forward use: ``transpose_b``
either way, no activation, no accumulate-into-c)."""

from __future__ import annotations

from typing import Optional

import torch

from .... import ops


def group_gemm_same_nk(
    a: torch.Tensor,
    b: torch.Tensor,
    cumsum_M: torch.Tensor,
    max_M: int,
    transpose_a: bool = False,
    transpose_b: bool = False,
    activation=None,
    save_activation: bool = False,
    c: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Rows ``[cumsum_M[g-1], cumsum_M[g])`` of ``a`` are multiplied by group ``g``'s matrix:
    ``b[g]`` is ``[N, K]`` when ``transpose_b`` else ``[K, N]``."""
    assert not transpose_a, "Transpose A not tested yet."
    assert a.dtype in [torch.bfloat16, torch.float16], a.dtype
    assert b.dtype in [torch.bfloat16, torch.float16], b.dtype
    assert a.device == b.device, f"a.device = {a.device}, b.device = {b.device}"
    assert len(cumsum_M) == b.shape[0]
    assert activation is None, f"Not implemented: activation is {activation}."
    assert not save_activation, "Can't save activation since activation type is None"
    assert a.is_contiguous() and b.is_contiguous(), "Not implemented: Noncontiguous input."
    if c is not None:
        raise NotImplementedError("accumulating into c is a backward-pass feature and is not built")
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise NotImplementedError("the grouped GEMM is built for bfloat16")
    w = b if transpose_b else b.transpose(1, 2).contiguous()  # [G, N, K]
    G = w.shape[0]
    rows = a.shape[0]
    # Rebuild per-row group ids from the cumulative sizes, then route them like expert indices
    # (k = 1): rows of a group are already contiguous, so the stable ranks are the identity.
    bounds = cumsum_M.to(torch.int64)
    group_of_row = torch.searchsorted(bounds, torch.arange(rows, device=a.device, dtype=torch.int64), right=True)
    group_of_row = group_of_row.clamp_(max=G - 1).to(torch.int32).view(rows, 1)
    routing = ops.moe_route(group_of_row, G, bm=ops.moe_tile_rows(rows, wide_ok=w.shape[-1] % 64 == 0, top_k=1, num_experts=G))
    return ops.moe_gemm(a, w, routing)
