"""Oracle (test infrastructure): router, routing integers and the fused-order expert MLP on the CPU."""

from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F


def router_ref(router_logits: torch.Tensor, top_k: int, renorm: bool = True, out_dtype=torch.bfloat16):
    """fp32 softmax -> top-k (descending; ties: lower expert index first) -> renormalise -> cast
    (vexact/models/qwen3_moe/modeling_qwen3_moe.py:128-134). ``torch.topk`` leaves tie order open;
    a stable descending sort fixes it."""
    probs = F.softmax(router_logits, dim=1, dtype=torch.float32)
    order = torch.sort(probs, dim=-1, descending=True, stable=True).indices[:, :top_k]
    w = probs.gather(-1, order)
    if renorm:
        w = w / w.sum(dim=-1, keepdim=True)
    return w.to(out_dtype), order


def router_weights_for(router_logits: torch.Tensor, idx: torch.Tensor, renorm: bool = True, out_dtype=torch.bfloat16):
    """Routing weights for a GIVEN expert choice (same softmax / renormalise / cast as router_ref).
    Used when a test forces the oracle onto the routing another implementation chose at a near-tie."""
    probs = F.softmax(router_logits, dim=1, dtype=torch.float32)
    w = probs.gather(-1, idx.to(torch.int64))
    if renorm:
        w = w / w.sum(dim=-1, keepdim=True)
    return w.to(out_dtype)


def routing_integers_ref(selected_experts, num_experts: int):
    """splits, cumulative offsets, stable expert-major rank of every (token, slot), and the inverse
    order (vexact/batch_invariant_ops/group_gemm/kernel/moe.py:26-49 histogram;
    vexact/batch_invariant_ops/fused_moe.py:43 and :268-292)."""
    idx = np.asarray(selected_experts.cpu()).astype(np.int64)
    T, k = idx.shape
    flat = idx.reshape(-1)
    splits = np.bincount(flat, minlength=num_experts).astype(np.int32)
    cu = np.concatenate([[0], np.cumsum(splits)]).astype(np.int32)
    sorted_order = np.argsort(flat, kind="stable")
    scatter_index = np.argsort(sorted_order, kind="stable").astype(np.int32).reshape(T, k)
    return {
        "splits": splits,
        "cu": cu,
        "scatter_index": scatter_index,
        "sorted_flat": sorted_order.astype(np.int32),
        "sorted_token": (sorted_order // k).astype(np.int32),
    }


def tile_table_ref(splits, bm: int):
    """Row tiles of at most ``bm`` rows per expert, experts ascending (this build's own table)."""
    groups, row0, rows = [], [], []
    base = 0
    for e, c in enumerate(np.asarray(splits)):
        for off in range(0, int(c), bm):
            groups.append(e)
            row0.append(base + off)
            rows.append(min(bm, int(c) - off))
        base += int(c)
    return np.array(groups, np.int32), np.array(row0, np.int32), np.array(rows, np.int32)


def _bf(x):
    return x.to(torch.bfloat16)


def fused_moe_ref(hidden, routing_weights, selected_experts, gate_w, up_w, down_w):
    """Fused-order expert MLP (vexact/batch_invariant_ops/fused_moe.py:38-102 with
    group_gemm/kernel/moe.py:84-128): bf16 gate and up projections, ``bf16(silu(g))``, ``* u``,
    ``* w_slot`` (each rounded to bf16), bf16 down projection, fp32 sum over the token's slots in slot
    order, one final rounding. ``gate_w/up_w [E,I,H]``, ``down_w [E,H,I]``."""
    x = _bf(hidden)
    w = _bf(routing_weights)
    T, k = selected_experts.shape
    H = x.shape[1]
    slot_out = torch.zeros(T, k, H, dtype=torch.float32)
    sel = selected_experts.to(torch.int64)
    for e in torch.unique(sel).tolist():
        tok, slot = torch.nonzero(sel == e, as_tuple=True)
        xe = x[tok].float()
        g = _bf(xe @ gate_w[e].float().t())
        u = _bf(xe @ up_w[e].float().t())
        a = _bf(F.silu(g.float()))
        h = _bf(a.float() * u.float())
        hw = _bf(h.float() * w[tok, slot].float().unsqueeze(1))
        o = _bf(hw.float() @ down_w[e].float().t())
        slot_out[tok, slot] = o.float()
    acc = torch.zeros(T, H, dtype=torch.float32)
    for i in range(k):
        acc = acc + slot_out[:, i]
    return _bf(acc)


def hf_eager_moe_ref(hidden, routing_weights, selected_experts, gate_w, up_w, down_w):
    """HuggingFace-style eager experts: routing weight applied after the down projection and
    outputs accumulated in bf16 in expert order (the form of
    tests/batch_invariant_ops/test_naive_moe.py:45-86). Reported beside the fused order, not a
    parity target."""
    x = _bf(hidden)
    out = torch.zeros_like(x)
    sel = selected_experts.to(torch.int64)
    for e in range(gate_w.shape[0]):
        tok, slot = torch.nonzero(sel == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        xe = x[tok]
        g = _bf(xe.float() @ gate_w[e].float().t())
        u = _bf(xe.float() @ up_w[e].float().t())
        h = _bf(_bf(F.silu(g.float())).float() * u.float())
        o = _bf(h.float() @ down_w[e].float().t())
        o = _bf(o.float() * _bf(routing_weights)[tok, slot].float().unsqueeze(1))
        out.index_add_(0, tok, o)
    return out


def fused_moe_backward_ref(hidden, routing_weights, selected_experts, gate_w, up_w, down_w, grad_out):
    """Backward of the fused expert MLPs with the reference's formulas and bf16 intermediates
    (FusedMoeExpertFunction.backward, vexact/batch_invariant_ops/fused_moe.py:126-265): per
    (token, slot) row of expert ``e``: ``g = x Wg^T``, ``u = x Wu^T``, ``a = silu(g)``, ``act = a u``,
    ``hw = act w``; ``d_hw = dY Wd``, ``dWd += dY^T hw``, ``d_act = d_hw w``, ``dw = sum(act d_hw)``,
    ``d_a = d_act u``, ``d_u = a d_act``, ``d_g = silu'(g) d_a``, ``dx += d_g Wg + d_u Wu``,
    ``dWg += d_g^T x``, ``dWu += d_u^T x``. Returns (d_routing_weights, d_hidden, dWg, dWu, dWd)."""
    x, w, dy = _bf(hidden), _bf(routing_weights), _bf(grad_out)
    T, k = selected_experts.shape
    sel = selected_experts.to(torch.int64)
    d_w = torch.zeros(T, k, dtype=torch.float32)
    d_x_slots = torch.zeros(T, k, x.shape[1], dtype=torch.float32)
    d_g_w, d_u_w, d_d_w = (torch.zeros_like(t, dtype=torch.float32) for t in (gate_w, up_w, down_w))
    for e in torch.unique(sel).tolist():
        tok, slot = torch.nonzero(sel == e, as_tuple=True)
        xe, dye = x[tok].float(), dy[tok].float()
        g = _bf(xe @ gate_w[e].float().t())
        u = _bf(xe @ up_w[e].float().t())
        a = _bf(F.silu(g.float()))
        act = _bf(a.float() * u.float())
        ws = w[tok, slot].float().unsqueeze(1)
        hw = _bf(act.float() * ws)
        d_hw = _bf(dye @ down_w[e].float())
        d_d_w[e] = dye.t() @ hw.float()
        d_act = _bf(d_hw.float() * ws)
        d_w[tok, slot] = _bf((act.float() * d_hw.float()).sum(-1)).float()
        d_a = _bf(d_act.float() * u.float())
        d_u = _bf(a.float() * d_act.float())
        sg = torch.sigmoid(g.float())
        d_g = _bf(d_a.float() * sg * (1 + g.float() * (1 - sg)))
        d_x_slots[tok, slot] = _bf(d_g.float() @ gate_w[e].float()).float() + _bf(d_u.float() @ up_w[e].float()).float()
        d_g_w[e] = d_g.float().t() @ xe
        d_u_w[e] = d_u.float().t() @ xe
    d_x = torch.zeros(T, x.shape[1], dtype=torch.float32)
    for i in range(k):
        d_x = d_x + _bf(d_x_slots[:, i]).float()
    return _bf(d_w), _bf(d_x), _bf(d_g_w), _bf(d_u_w), _bf(d_d_w)
