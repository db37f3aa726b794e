"""Qwen3-MoE sparse block on the HIP kernels: the patch points of
``vexact/models/qwen3_moe/modeling_qwen3_moe.py`` (``Qwen3MoeExperts`` :42-100, ``moe_block_init`` :103-116,
``moe_block_forward`` :119-145, ``apply_qwen3_moe_patches`` :291-302).

The experts keep the reference's parameter names and stacked layout (``gate_up_proj [E, 2I, H]`` with the
gate rows first, ``down_proj [E, H, I]``), so weight synchronisation from an actor needs no renaming. The
router (softmax in fp32 -> top-k -> renormalise -> cast) runs as one kernel; the expert MLPs are
``fused_moe_forward``. There is no CPU path: tensors off the GPU raise. Checkpoint loading
(``load_qwen3_moe_weights``) belongs to the reference's model loader and is not rebuilt here.
"""

from __future__ import annotations

from types import SimpleNamespace
from typing import Optional

import torch
import torch.nn as nn

from ... import ops
from ...batch_invariant_ops.fused_moe import fused_moe_forward

_ORIGINAL = None  # (Qwen3MoeSparseMoeBlock.__init__, .forward) while the patches are applied


class Qwen3MoeExperts(nn.Module):
    """All experts of a layer in two stacked parameters."""

    def __init__(self, config):
        super().__init__()
        self.num_experts = config.num_experts
        self.hidden_dim = config.hidden_size
        self.intermediate_size = config.moe_intermediate_size
        if getattr(config, "hidden_act", "silu") != "silu":
            raise ValueError(f"the fused expert kernels implement silu, got hidden_act={config.hidden_act!r}")
        self.gate_up_proj = nn.Parameter(torch.empty(self.num_experts, 2 * self.intermediate_size, self.hidden_dim))
        self.down_proj = nn.Parameter(torch.empty(self.num_experts, self.hidden_dim, self.intermediate_size))

        self._packed = None  # (packed gate_up, packed down, (data_ptr, version) of both parameters)
        # every path of this module that replaces or rewrites the parameters drops the copies
        self.register_load_state_dict_post_hook(lambda module, incompatible: module.invalidate_packed())

    def _weights_key(self):
        return (self.gate_up_proj.data_ptr(), self.gate_up_proj._version, self.down_proj.data_ptr(), self.down_proj._version)

    def pack_for_decode(self) -> None:
        """Keep fragment-order copies of both parameters for decode-sized steps (a second copy of the
        expert weights in HBM; opt-in).

        Contract: the copies are a snapshot. Whoever writes the parameters afterwards must call
        ``invalidate_packed()`` (or this method again) before the next forward; ``invalidate_packed_experts(model)``
        does it for every layer after a weight synchronisation. ``load_state_dict``, ``.to()`` / ``.cuda()`` and
        in-place tensor methods on the parameter (``mul_``, ``copy_`` ...) are noticed by the module itself. A write
        through ``param.data`` (what the reference's weight sync does, vexact/inferencer/model_loader.py:113) or a
        raw device copy leaves no trace a module could see, hence the explicit call."""
        if self.intermediate_size % 16 != 0 or self.gate_up_proj.dtype != torch.bfloat16:
            raise ValueError("packed expert weights need bf16 parameters and an intermediate size that is a multiple of 16")
        with torch.no_grad():
            self._packed = (ops.pack_expert_weights(self.gate_up_proj.detach()),
                            ops.pack_expert_weights(self.down_proj.detach()), self._weights_key())

    def invalidate_packed(self) -> None:
        """Forget the fragment-order copies: the next forward reads the parameters."""
        self._packed = None

    def _apply(self, fn, *args, **kwargs):  # .to() / .cuda() / .half(): new storage, the copies are void
        self._packed = None
        return super()._apply(fn, *args, **kwargs)

    def forward(self, hidden_states: torch.Tensor, expert_idx: Optional[int] = None,
                routing_weights: Optional[torch.Tensor] = None, selected_experts: Optional[torch.Tensor] = None):
        if expert_idx is not None:  # one expert as a dense SwiGLU MLP
            inter = self.intermediate_size
            w = self.gate_up_proj[expert_idx]
            x = hidden_states.reshape(-1, self.hidden_dim)
            return ops.swiglu_mlp(x, w[:inter], w[inter:], self.down_proj[expert_idx]).reshape(hidden_states.shape)
        assert routing_weights is not None and selected_experts is not None, (
            "routing_weights and selected_experts must be provided when expert_idx is None"
        )
        packed = None
        if self._packed is not None:
            if self._packed[2] == self._weights_key():
                packed = self._packed[:2]
            else:
                self._packed = None  # stale: the parameters were written since
        return fused_moe_forward(
            num_experts=self.num_experts, routing_weights=routing_weights, selected_experts=selected_experts,
            hidden_states=hidden_states, fc1_1_weight=None, fc1_2_weight=None, fc2_weight=self.down_proj,
            fc1_1_2_weight=self.gate_up_proj, packed_weights=packed,
        )


def moe_block_init(self, config):
    """Replacement for ``Qwen3MoeSparseMoeBlock.__init__``: a plain linear router and fused experts."""
    nn.Module.__init__(self)
    self.num_experts = config.num_experts
    self.top_k = config.num_experts_per_tok
    self.norm_topk_prob = config.norm_topk_prob
    self._fused_config = SimpleNamespace(
        num_experts=config.num_experts, hidden_size=config.hidden_size,
        moe_intermediate_size=config.moe_intermediate_size, hidden_act=getattr(config, "hidden_act", "silu"),
    )
    self.gate = nn.Linear(config.hidden_size, config.num_experts, bias=False)
    self.experts = Qwen3MoeExperts(config)


def moe_block_forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
    """Replacement for ``Qwen3MoeSparseMoeBlock.forward``; returns the hidden states only."""
    if not isinstance(self.experts, Qwen3MoeExperts):
        raise AssertionError(
            "Qwen3-MoE experts are not fused. Ensure apply_qwen3_moe_patches() is called before loading the model."
        )
    batch_size, sequence_length, hidden_dim = hidden_states.shape
    x = hidden_states.view(-1, hidden_dim)
    router_logits = self.gate(x)  # aten::mm -> the batch-invariant GEMM when the mode is on
    routing_weights, selected_experts = ops.router_topk(
        router_logits, self.top_k, renorm=bool(self.norm_topk_prob), out_dtype=x.dtype, index_dtype=torch.int64)
    out = self.experts(x, routing_weights=routing_weights, selected_experts=selected_experts)
    return out.reshape(batch_size, sequence_length, hidden_dim)


def invalidate_packed_experts(model: nn.Module) -> int:
    """Drop the fragment-order expert copies of every layer of ``model``; call once after a weight
    synchronisation that wrote the parameters. Returns the number of expert containers visited."""
    n = 0
    for m in model.modules():
        if isinstance(m, Qwen3MoeExperts):
            m.invalidate_packed()
            n += 1
    return n


def apply_qwen3_moe_patches() -> None:
    """Swap the HuggingFace block's constructor and forward (idempotent)."""
    global _ORIGINAL
    if _ORIGINAL is not None:
        return
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeSparseMoeBlock

    _ORIGINAL = (Qwen3MoeSparseMoeBlock.__init__, Qwen3MoeSparseMoeBlock.forward)
    Qwen3MoeSparseMoeBlock.__init__ = moe_block_init
    Qwen3MoeSparseMoeBlock.forward = moe_block_forward


def remove_qwen3_moe_patches() -> None:
    """Put the HuggingFace block's own constructor and forward back (blocks built meanwhile keep their fused
    experts and stop working with the original forward; meant for tests and tools that need both forms)."""
    global _ORIGINAL
    if _ORIGINAL is None:
        return
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeSparseMoeBlock

    Qwen3MoeSparseMoeBlock.__init__, Qwen3MoeSparseMoeBlock.forward = _ORIGINAL
    _ORIGINAL = None
