"""Fused MoE expert forward on the HIP kernels.

Mirrors ``fused_moe_forward`` of ``vexact/batch_invariant_ops/fused_moe.py:459-487`` and the
``fc1_1_2_weight=`` form the Qwen3-MoE patch calls
(``vexact/models/qwen3_moe/modeling_qwen3_moe.py:89-100``). Arithmetic follows
``FusedMoeExpertFunction.forward`` (fused_moe.py:24-102): bf16 gate/up projections, bf16
``silu(g) * u``, routing weight applied before the down projection, fp32 sum over a token's slots
in slot order. The backward (``FusedMoeExpertFunction.backward``, fused_moe.py:126-265) recomputes
the gate / up projections with the forward's grouped kernel and runs the data- and weight-gradient
products on the grouped kernels of ``csrc/moe_bwd.hip``; only the forward has to match the rollout bit
for bit.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import ops
from .group_gemm.kernel.group_gemm import group_gemm_same_nk
from .group_gemm.kernel.moe import expert_histogram, moe_gather, moe_scatter


def _split_weights(fc1_1_weight, fc1_2_weight, fc1_1_2_weight):
    if fc1_1_2_weight is not None:
        two_i = fc1_1_2_weight.shape[1]
        assert two_i % 2 == 0, "fused gate/up weight must have an even number of rows per expert"
        inter = two_i // 2
        return fc1_1_2_weight[:, :inter, :], fc1_1_2_weight[:, inter:, :]
    assert fc1_1_weight is not None and fc1_1_weight.shape == fc1_1_weight.shape
    assert fc1_2_weight is not None and fc1_1_weight.shape == fc1_2_weight.shape
    if fc1_1_weight.stride() != fc1_2_weight.stride():
        fc1_1_weight, fc1_2_weight = fc1_1_weight.contiguous(), fc1_2_weight.contiguous()
    return fc1_1_weight, fc1_2_weight


class FusedMoeExpertFunction(torch.autograd.Function):
    """Forward on the HIP kernels (bit-identical to the inference path); backward with the formulas
    of the reference's ``FusedMoeExpertFunction.backward`` (fused_moe.py:126-265). Gradients for the
    routing weights, the hidden states and the three expert weights."""

    @staticmethod
    def forward(ctx, num_experts, routing_weights, selected_experts, hidden_states, gate_w, up_w, down_w):
        x = hidden_states.reshape(-1, hidden_states.shape[-1])
        out = ops.fused_moe(x, routing_weights.reshape(x.shape[0], -1), selected_experts.reshape(x.shape[0], -1),
                            gate_w, up_w, down_w, num_experts)
        ctx.num_experts = num_experts
        ctx.save_for_backward(routing_weights, selected_experts, hidden_states, gate_w, up_w, down_w)
        return out.reshape(hidden_states.shape)

    @staticmethod
    def backward(ctx, grad_output):
        routing_weights, selected_experts, hidden_states, gate_w, up_w, down_w = ctx.saved_tensors
        E = ctx.num_experts
        H = hidden_states.shape[-1]
        x = hidden_states.reshape(-1, H)
        T, k = x.shape[0], selected_experts.reshape(x.shape[0], -1).shape[1]
        dy = grad_output.reshape(-1, H).to(torch.bfloat16)
        # 256-row expert tiles (the wide kernels) when every contraction depth is a multiple of 64
        wide_ok = H % 64 == 0 and gate_w.shape[1] % 64 == 0 and up_w.shape[1] % 64 == 0
        r = ops.moe_route(selected_experts.reshape(T, k), E, bm=ops.moe_tile_rows(T, wide_ok=wide_ok, top_k=k, num_experts=E))
        # recomputed with the forward's kernels, so these are the values the forward used
        g = ops.moe_gemm(x, gate_w, r, row_src=r.sorted_token)
        u = ops.moe_gemm(x, up_w, r, row_src=r.sorted_token)
        # grouped products on the HIP kernels; the row gathers x[tok], dy[tok] happen inside them
        d_hw = ops.moe_gemm_nn(dy, down_w, r, a_src=r.sorted_token)                # dgrad of the down projection
        if g.shape[1] % 8 == 0 and routing_weights.dtype == torch.bfloat16:
            # silu, its derivative, the routing-weight gradient and the scatter back to (token, slot) in one launch
            hw, d_g, d_u, grad_rw = ops.moe_swiglu_backward(g, u, d_hw, routing_weights.reshape(T, k), r.sorted_flat)
        else:
            flat = r.sorted_flat.long()                  # (token, slot) flat index of each sorted row
            a = torch.ops.aten.silu(g)
            act = a * u
            w_sorted = routing_weights.reshape(-1)[flat].unsqueeze(1)
            hw = act * w_sorted
            d_act = d_hw * w_sorted
            d_w_sorted = torch.sum(act * d_hw, dim=-1)
            grad_rw = torch.empty_like(d_w_sorted)
            grad_rw[flat] = d_w_sorted
            d_a, d_u = d_act * u, a * d_act
            d_g = torch.ops.aten.silu_backward(d_a, g)
        d_d_w = ops.moe_gemm_tn(dy, hw, r.cu, E, dy_src=r.sorted_token) if ctx.needs_input_grad[6] else None
        d_xs = ops.moe_gemm_nn(d_g, gate_w, r, a2=d_u, w2=up_w)
        d_g_w = ops.moe_gemm_tn(d_g, x, r.cu, E, x_src=r.sorted_token) if ctx.needs_input_grad[4] else None
        d_u_w = ops.moe_gemm_tn(d_u, x, r.cu, E, x_src=r.sorted_token) if ctx.needs_input_grad[5] else None
        d_x = ops.moe_gather(d_xs, r.scatter_index)
        return (None, grad_rw.reshape(routing_weights.shape).to(routing_weights.dtype), None,
                d_x.reshape(hidden_states.shape), d_g_w, d_u_w, d_d_w)


class FusedMoeStackedFunction(torch.autograd.Function):
    """``FusedMoeExpertFunction`` for gate and up projections stacked in one tensor ``[E, 2I, H]`` (the layout of
    ``Qwen3MoeExperts.gate_up_proj``; not in the reference, which slices the stacked parameter and lets autograd
    scatter the two gradients back into a zero-filled ``[E, 2I, H]`` each). Same forward; the backward treats
    gate and up as one projection of width 2 I: one recompute launch, one data-gradient product over K = 2 I
    (the accumulation chain of ``d_g W_gate + d_u W_up``, so the same bits) and one weight-gradient launch that
    writes the stacked gradient directly."""

    @staticmethod
    def forward(ctx, num_experts, routing_weights, selected_experts, hidden_states, gate_up_w, down_w):
        x = hidden_states.reshape(-1, hidden_states.shape[-1])
        inter = gate_up_w.shape[1] // 2
        out = ops.fused_moe(x, routing_weights.reshape(x.shape[0], -1), selected_experts.reshape(x.shape[0], -1),
                            gate_up_w[:, :inter], gate_up_w[:, inter:], down_w, num_experts)
        ctx.num_experts = num_experts
        ctx.save_for_backward(routing_weights, selected_experts, hidden_states, gate_up_w, down_w)
        return out.reshape(hidden_states.shape)

    @staticmethod
    def backward(ctx, grad_output):
        routing_weights, selected_experts, hidden_states, gate_up_w, down_w = ctx.saved_tensors
        E = ctx.num_experts
        H, inter = hidden_states.shape[-1], gate_up_w.shape[1] // 2
        x = hidden_states.reshape(-1, H)
        T, k = x.shape[0], selected_experts.reshape(x.shape[0], -1).shape[1]
        dy = grad_output.reshape(-1, H).to(torch.bfloat16)
        wide_ok = H % 64 == 0 and inter % 64 == 0
        r = ops.moe_route(selected_experts.reshape(T, k), E, bm=ops.moe_tile_rows(T, wide_ok=wide_ok, top_k=k, num_experts=E))
        gu = ops.moe_gemm(x, gate_up_w, r, row_src=r.sorted_token)                 # [T k, 2I]: gate | up, as the forward
        d_hw = ops.moe_gemm_nn(dy, down_w, r, a_src=r.sorted_token)
        d_gu = ops._empty_like(gu)
        hw, _, _, grad_rw = ops.moe_swiglu_backward(gu[:, :inter], gu[:, inter:], d_hw, routing_weights.reshape(T, k),
                                                    r.sorted_flat, d_g_out=d_gu[:, :inter], d_u_out=d_gu[:, inter:])
        d_d_w = ops.moe_gemm_tn(dy, hw, r.cu, E, dy_src=r.sorted_token) if ctx.needs_input_grad[5] else None
        d_xs = ops.moe_gemm_nn(d_gu, gate_up_w, r)
        d_gu_w = ops.moe_gemm_tn(d_gu, x, r.cu, E, x_src=r.sorted_token) if ctx.needs_input_grad[4] else None
        d_x = ops.moe_gather(d_xs, r.scatter_index)
        return (None, grad_rw.reshape(routing_weights.shape).to(routing_weights.dtype), None,
                d_x.reshape(hidden_states.shape), d_gu_w, d_d_w)


def fused_moe_forward(
    num_experts: int,
    routing_weights: torch.Tensor,
    selected_experts: torch.Tensor,
    hidden_states: torch.Tensor,
    fc1_1_weight: Optional[torch.Tensor],
    fc1_2_weight: Optional[torch.Tensor],
    fc2_weight: torch.Tensor,
    fc1_1_2_weight: Optional[torch.Tensor] = None,
    packed_weights: Optional[tuple] = None,
    residual: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``hidden_states [T,H]``, ``routing_weights/selected_experts [T,k]``; expert weights either as
    ``fc1_1_weight`` (gate) + ``fc1_2_weight`` (up), each ``[E,I,H]``, or fused ``fc1_1_2_weight [E,2I,H]``
    (gate rows first); ``fc2_weight [E,H,I]``. Returns ``[T,H]`` bf16. ``packed_weights`` (not in the
    reference; inference only): fragment-order copies of the same weights, ``(ops.pack_expert_weights(
    fc1_1_2_weight), ops.pack_expert_weights(fc2_weight))``, streamed instead at decode sizes. ``residual`` (not
    in the reference; bf16, the shape of ``hidden_states``): returns ``residual + output`` with the rounding of a
    separate bf16 add, inside the combine kernel."""
    routing_weights = routing_weights.bfloat16()
    hidden_states = hidden_states.bfloat16()
    gate_w, up_w = _split_weights(fc1_1_weight, fc1_2_weight, fc1_1_2_weight)
    gate_w, up_w, down_w = gate_w.bfloat16(), up_w.bfloat16(), fc2_weight.bfloat16()
    if gate_w.stride(2) != 1 or up_w.stride() != gate_w.stride():
        gate_w, up_w = gate_w.contiguous(), up_w.contiguous()
    if down_w.stride(2) != 1:
        down_w = down_w.contiguous()
    shape = hidden_states.shape
    if torch.is_grad_enabled() and any(t.requires_grad for t in (routing_weights, hidden_states, gate_w, up_w, down_w)):
        stacked = fc1_1_2_weight
        if (stacked is not None and stacked.dtype == torch.bfloat16 and stacked.stride(2) == 1
                and stacked.shape[1] % 16 == 0 and stacked.shape[2] % 8 == 0):
            out = FusedMoeStackedFunction.apply(num_experts, routing_weights, selected_experts, hidden_states, stacked, down_w)
            return out if residual is None else residual + out
        out = FusedMoeExpertFunction.apply(num_experts, routing_weights, selected_experts, hidden_states, gate_w, up_w,
                                           down_w)
        return out if residual is None else residual + out
    x = hidden_states.reshape(-1, shape[-1])
    res = None
    if residual is not None:
        res = residual.reshape(-1, shape[-1])
        if res.dtype != torch.bfloat16 or res.stride(1) != 1 or res.shape != x.shape:
            raise ValueError("residual must be a bf16 tensor of the shape of hidden_states, contiguous in its last dim")
    out = ops.fused_moe(
        x, routing_weights.reshape(x.shape[0], -1), selected_experts.reshape(x.shape[0], -1), gate_w, up_w, down_w,
        num_experts, packed=packed_weights, residual=res,
    )
    return out.reshape(shape)


def fused_moe_forward_unfused(
    num_experts: int,
    routing_weights: torch.Tensor,
    selected_experts: torch.Tensor,
    hidden_states: torch.Tensor,
    fc1_1_weight: torch.Tensor,
    fc1_2_weight: torch.Tensor,
    fc2_weight: torch.Tensor,
) -> torch.Tensor:
    """The same computation step by step through the public helpers (histogram, stable ranks,
    scatter, three grouped GEMMs, elementwise glue in torch, gather), as the reference's
    ``FusedMoeExpertFunction.forward`` lays it out. Must match ``fused_moe_forward`` bit for bit."""
    routing_weights = routing_weights.bfloat16()
    hidden_states = hidden_states.bfloat16()
    splits = expert_histogram(selected_experts, num_experts)
    scatter_index = selected_experts.flatten().argsort(stable=True).argsort().int().view(selected_experts.shape)
    scatter_output = moe_scatter(hidden_states, scatter_index)
    cumsum_t = torch.cumsum(splits, dim=0)
    max_m = scatter_output.shape[0]
    g = group_gemm_same_nk(scatter_output, fc1_1_weight, cumsum_t, max_m, transpose_b=True)
    u = group_gemm_same_nk(scatter_output, fc1_2_weight, cumsum_t, max_m, transpose_b=True)
    act = torch.ops.aten.silu(g) * u
    w = routing_weights.reshape(-1, 1)
    w_sorted = torch.empty_like(w)
    w_sorted[scatter_index.flatten().long()] = w
    hw = act * w_sorted
    o = group_gemm_same_nk(hw, fc2_weight, cumsum_t, max_m, transpose_b=True)
    return moe_gather(o, scatter_index).reshape(hidden_states.shape)
