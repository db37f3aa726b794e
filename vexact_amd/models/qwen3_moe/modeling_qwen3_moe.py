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
                routing_weights: Optional[torch.Tensor] = None, selected_experts: Optional[torch.Tensor] = None,
                residual: Optional[torch.Tensor] = None):
        if expert_idx is not None:  # one expert as a dense SwiGLU MLP
            assert residual is None
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
            fc1_1_2_weight=self.gate_up_proj, packed_weights=packed, residual=residual,
        )


class RouterTopKFunction(torch.autograd.Function):
    """``ops.router_topk`` with a gradient for the router logits, for the training side. The reference's block
    runs softmax -> top-k -> renormalise -> cast as tensor operations (modeling_qwen3_moe.py:128-134), which
    autograd differentiates; here the forward stays the one kernel of the rollout (same bits) and the backward
    applies the derivative of those operations to the recomputed fp32 softmax."""

    @staticmethod
    def forward(ctx, router_logits, top_k, renorm, out_dtype):
        weights, selected = ops.router_topk(router_logits, top_k, renorm=renorm, out_dtype=out_dtype, index_dtype=torch.int64)
        ctx.save_for_backward(router_logits, selected)
        ctx.renorm = renorm
        ctx.mark_non_differentiable(selected)
        return weights, selected

    @staticmethod
    def backward(ctx, d_weights, _):
        router_logits, selected = ctx.saved_tensors
        if router_logits.shape[-1] <= 512 and selected.shape[-1] <= 64 and router_logits.dtype in (torch.float32, torch.bfloat16):
            return ops.router_topk_backward(router_logits, selected, d_weights, ctx.renorm), None, None, None
        p = torch.softmax(router_logits.float(), dim=-1)
        d_sel = d_weights.float()
        if ctx.renorm:
            sel = p.gather(-1, selected)
            s = sel.sum(-1, keepdim=True)
            d_sel = (d_sel - (d_sel * (sel / s)).sum(-1, keepdim=True)) / s
        d_p = torch.zeros_like(p).scatter_(-1, selected, d_sel)
        d_logits = p * (d_p - (d_p * p).sum(-1, keepdim=True))
        return d_logits.to(router_logits.dtype), None, None, None


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


def moe_block_forward(self, hidden_states: torch.Tensor, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Replacement for ``Qwen3MoeSparseMoeBlock.forward``; returns the hidden states only. ``residual`` (not in
    the reference): the block returns ``residual + output``, added inside the combine kernel."""
    if not isinstance(self.experts, Qwen3MoeExperts):
        raise AssertionError(
            "Qwen3-MoE experts are not fused. Ensure apply_qwen3_moe_patches() is called before loading the model."
        )
    batch_size, sequence_length, hidden_dim = hidden_states.shape
    x = hidden_states.view(-1, hidden_dim)
    router_logits = self.gate(x)  # aten::mm -> the batch-invariant GEMM when the mode is on
    if torch.is_grad_enabled() and router_logits.requires_grad:
        routing_weights, selected_experts = RouterTopKFunction.apply(router_logits, self.top_k, bool(self.norm_topk_prob), x.dtype)
    else:
        routing_weights, selected_experts = ops.router_topk(
            router_logits, self.top_k, renorm=bool(self.norm_topk_prob), out_dtype=x.dtype, index_dtype=torch.int64)
    res = None if residual is None else residual.reshape(-1, hidden_dim)
    out = self.experts(x, routing_weights=routing_weights, selected_experts=selected_experts, residual=res)
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


class RmsNormFunction(torch.autograd.Function):
    """The fused RMSNorm with a backward, so that a trainer's forward runs the kernel the rollout ran (which has
    the bits of the tensor-operation forward under batch-invariant mode). Backward: the RMSNorm derivative,
    ``d_x = inv (d_h - h mean(d_h h))`` with ``h = x inv``, ``d_h = d_y w``, ``d_w = sum d_y r(h)``, in fp32: one
    kernel plus a small reduction (``ops.rms_norm_backward``), tensor operations for rows it does not take."""

    @staticmethod
    def forward(ctx, hidden_states, weight, eps):
        ctx.save_for_backward(hidden_states, weight)
        ctx.eps = eps
        return ops.rms_norm(hidden_states, weight, eps, hf_two_rounding=True)

    @staticmethod
    def backward(ctx, d_y):
        x, w = ctx.saved_tensors
        n = x.shape[-1]
        if n % 8 == 0 and n <= 8192 and w.dtype == x.dtype:
            d_x, d_w = ops.rms_norm_backward(x, w, d_y, ctx.eps, hf_two_rounding=True)
            return (d_x if ctx.needs_input_grad[0] else None), (d_w if ctx.needs_input_grad[1] else None), None
        x32, dy32 = x.float(), d_y.float()
        inv = torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + ctx.eps)
        h = x32 * inv
        d_w = None
        if ctx.needs_input_grad[1]:
            d_w = (dy32 * h.to(x.dtype).float()).reshape(-1, x.shape[-1]).sum(0).to(w.dtype)
        d_x = None
        if ctx.needs_input_grad[0]:
            d_h = dy32 * w.float()
            d_x = (inv * (d_h - h * (d_h * h).mean(-1, keepdim=True))).to(x.dtype)
        return d_x, d_w, None


def fused_rms_norm_forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
    """``Qwen3MoeRMSNorm.forward`` as one kernel. HuggingFace's forward (cast to fp32, ``pow(2).mean(-1)``, ``rsqrt``,
    two multiplies and two casts: eleven launches under batch-invariant mode) rounds ``x * rsqrt(var + eps)`` to
    the input dtype and then multiplies by the weight; ``ops.rms_norm(..., hf_two_rounding=True)`` keeps both
    roundings, the batch-invariant mean's summation order and the device's ``rsqrt`` (the operation ``torch.rsqrt``
    runs on the GPU), so the result has the bits of the original forward under batch-invariant mode (tested on
    rows of very different magnitudes). With autograd the same kernel runs (``RmsNormFunction``). Outside
    batch-invariant mode, off the GPU or with a weight of another dtype the original forward runs: the same
    bits again, hence a rollout and a trainer agree whether or not each of them takes the fused path."""
    from ...batch_invariant_ops import is_batch_invariant_mode_enabled

    w = self.weight
    if (hidden_states.is_cuda and hidden_states.dtype in (torch.bfloat16, torch.float16) and w.dtype == hidden_states.dtype
            and is_batch_invariant_mode_enabled()):
        if torch.is_grad_enabled() and (hidden_states.requires_grad or w.requires_grad):
            return RmsNormFunction.apply(hidden_states, w, self.variance_epsilon)
        return ops.rms_norm(hidden_states, w, self.variance_epsilon, hf_two_rounding=True)
    return _ORIGINAL_NORM(self, hidden_states)


_ORIGINAL_NORM = None  # Qwen3MoeRMSNorm.forward while the fused form is patched in
_ORIGINAL_ROPE = None  # the module's apply_rotary_pos_emb while the fused form is patched in


class RopeFunction(torch.autograd.Function):
    """``ops.rope`` with its backward. ``y = x cos + R(x) sin`` with ``R(x) = (-x2, x1)``; ``R`` is antisymmetric and
    both halves of HuggingFace's ``sin`` are equal, so ``d_x = d_y cos - R(d_y) sin``: the same kernel on ``-sin``, with
    the bf16 roundings autograd's tensor operations would make."""

    @staticmethod
    def forward(ctx, x, cos, sin):
        ctx.save_for_backward(cos, sin)
        return ops.rope(x, cos, sin)

    @staticmethod
    def backward(ctx, d_y):
        cos, sin = ctx.saved_tensors
        g = d_y if (d_y.stride(2) == 1 and d_y.stride(0) % 4 == 0 and d_y.stride(1) % 4 == 0) else d_y.contiguous()
        return ops.rope(g, cos, -sin), None, None


def fused_apply_rotary_pos_emb(q, k, cos, sin, *args, unsqueeze_dim: int = 1, **kwargs):
    """``apply_rotary_pos_emb`` of HuggingFace's Qwen3-MoE modeling file as one launch per tensor instead of five
    (multiply, negate, concatenate, multiply, add). ``q`` / ``k`` are ``[B, heads, T, D]`` views of ``[B, T, heads, D]``
    projections, ``cos`` / ``sin`` ``[B, T, D]``. Elementwise with the same bf16 roundings, so the bits do not change
    in any mode; with autograd the same kernel runs in both directions (``RopeFunction``; ``cos`` / ``sin`` get no
    gradient, they come from position ids); other layouts or dtypes fall through to the original."""
    def fits(x):
        return (x.dim() == 4 and x.is_cuda and x.dtype == torch.bfloat16 and x.stride(3) == 1 and x.shape[3] % 8 == 0
                and (x.shape[0] == 1 or x.stride(0) == x.shape[2] * x.stride(2)) and x.stride(1) % 4 == 0 and x.stride(2) % 4 == 0)

    if (not args and not kwargs and unsqueeze_dim == 1 and fits(q) and fits(k) and cos.dim() == 3 and cos.dtype == torch.bfloat16
            and sin.dtype == torch.bfloat16 and cos.shape == sin.shape and cos.shape[0] == q.shape[0] == k.shape[0]
            and cos.shape[1] == q.shape[2] == k.shape[2] and cos.shape[2] == q.shape[3] == k.shape[3]
            and not (torch.is_grad_enabled() and (cos.requires_grad or sin.requires_grad))):
        B, _, T, D = q.shape
        c2, s2 = cos.reshape(B * T, D), sin.reshape(B * T, D)

        def one(x):
            H = x.shape[1]
            rows = x.transpose(1, 2)  # [B, T, H, D]
            flat = rows.as_strided((B * T, H, D), (rows.stride(1), rows.stride(2), 1), rows.storage_offset())
            if torch.is_grad_enabled() and x.requires_grad:
                return RopeFunction.apply(flat, c2, s2).view(B, T, H, D).transpose(1, 2)
            return ops.rope(flat, c2, s2).view(B, T, H, D).transpose(1, 2)

        return one(q), one(k)
    return _ORIGINAL_ROPE(q, k, cos, sin, *args, unsqueeze_dim=unsqueeze_dim, **kwargs)


_ORIGINAL_ATTN = None  # Qwen3MoeAttention.forward while the fused form is patched in


def _qkv_modules(model):
    for m in model.modules():
        if all(hasattr(m, n) and hasattr(getattr(m, n), "weight") for n in ("q_proj", "k_proj", "v_proj")):
            yield m


def fuse_qkv_weights(model) -> int:
    """Load-time step, optional: give every attention module of ``model`` ONE tensor
    ``[q_proj.weight; k_proj.weight; v_proj.weight]`` and re-point the three parameters at row ranges of it. The
    fused attention forward then runs one projection instead of three (same bits: a row of a product depends on its
    own weight row only). There is still one copy of the weights in memory, and an in-place write to a parameter
    (``param.data.copy_``, what the reference's weight sync does, vexact/inferencer/model_loader.py:113) lands in the
    fused tensor. What changes for the caller, and why this is a call of its own and not a side effect of a forward:
    the three parameters share one storage afterwards, so ``safetensors.save_file(model.state_dict())`` refuses them
    (``save_model`` or ``unfuse_qkv_weights`` first), and anything that captured the old storages (exported IPC
    handles, flat-parameter or bucketed weight-sync buffers) no longer aliases the parameters: call this before
    such captures are made. Call it outside graph capture. Returns the number of modules fused."""
    n = 0
    with torch.inference_mode(False), torch.no_grad():  # these tensors become parameter storage: keep them out of inference mode
        for attn in _qkv_modules(model):
            ws = (attn.q_proj.weight, attn.k_proj.weight, attn.v_proj.weight)
            if len({w.dtype for w in ws}) != 1 or len({w.device for w in ws}) != 1 or len({w.shape[1] for w in ws}) != 1:
                continue
            fused = torch.cat([w.detach() for w in ws], dim=0)
            row = 0
            for w in ws:
                w.data = fused[row:row + w.shape[0]]
                row += w.shape[0]
            attn._vx_qkv_weight = fused
            n += 1
    return n


def unfuse_qkv_weights(model) -> int:
    """Undo ``fuse_qkv_weights``: every q / k / v parameter gets storage of its own again (a copy)."""
    n = 0
    with torch.inference_mode(False), torch.no_grad():
        for attn in _qkv_modules(model):
            if getattr(attn, "_vx_qkv_weight", None) is None:
                continue
            for proj in (attn.q_proj, attn.k_proj, attn.v_proj):
                proj.weight.data = proj.weight.data.clone()
            attn._vx_qkv_weight = None
            n += 1
    return n


def _fused_qkv_weight(attn) -> Optional[torch.Tensor]:
    """The tensor ``fuse_qkv_weights`` made for this module, if the three parameters still are its row ranges (a
    parameter that has been given new storage since is noticed by its address); else None. Never builds one."""
    fused = getattr(attn, "_vx_qkv_weight", None)
    if fused is None:
        return None
    row = 0
    for w in (attn.q_proj.weight, attn.k_proj.weight, attn.v_proj.weight):
        if w.data_ptr() != fused[row].data_ptr() or w.dtype != fused.dtype or w.stride(0) != fused.stride(0):
            return None
        row += w.shape[0]
    return fused if row == fused.shape[0] else None


def fused_attention_forward(self, hidden_states, position_embeddings, attention_mask=None, past_key_values=None, **kwargs):
    """``Qwen3MoeAttention.forward`` for a step over the paged cache as a few launches in front of the output
    projection instead of twelve: the q / k / v projections written side by side into one buffer (one launch on the
    concatenated weight when ``fuse_qkv_weights`` has been called on the model, else three; the parameters are never
    touched here), one kernel for the per-head q / k RMSNorm, the rotary embedding and the cache write
    (``ops.qk_norm_rope_store``; it computes what ``q_norm`` / ``k_norm``, ``apply_rotary_pos_emb`` and
    ``store_kvcache`` compute, rounding for rounding), the attention kernel, then ``o_proj``. A row of a product
    depends on its own weight row only, so the concatenated projection gives the three projections' bits. The cache
    layer is ``kwargs["layer_idx"]`` if given, else the module's, as in the registered attention function.
    Taken only under batch-invariant mode with a paged context,
    the registered attention function of this package, bf16 tensors of batch 1 and no autograd, bias, HuggingFace
    cache object or sliding window; anything else runs the original forward."""
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    from ...batch_invariant_ops import flash_attention_forward, flash_attn_varlen_func, is_batch_invariant_mode_enabled
    from ...batch_invariant_ops.kv_cache_context import get_kv_cache_context

    ctx = get_kv_cache_context()
    cos, sin = position_embeddings
    D = self.head_dim
    fits = (
        ctx is not None and ctx.is_paged_attn and past_key_values is None and not self.training
        and is_batch_invariant_mode_enabled() and not torch.is_grad_enabled()
        and hidden_states.is_cuda and hidden_states.dtype == torch.bfloat16 and hidden_states.dim() == 3
        and hidden_states.shape[0] == 1 and D in (64, 128) and getattr(self, "sliding_window", None) is None
        and self.q_proj.bias is None and self.k_proj.bias is None and self.v_proj.bias is None
        and self.q_proj.weight.dtype == torch.bfloat16 and self.q_norm.weight.dtype == torch.bfloat16
        and cos.dtype == torch.bfloat16 and sin.dtype == torch.bfloat16 and cos.shape == sin.shape
        and cos.shape == (1, hidden_states.shape[1], D) and cos.is_contiguous() and sin.is_contiguous()
        and ALL_ATTENTION_FUNCTIONS.get(self.config._attn_implementation) is flash_attention_forward
    )
    if not fits:
        return _ORIGINAL_ATTN(self, hidden_states, position_embeddings, attention_mask, past_key_values, **kwargs)
    layer_idx = int(kwargs["layer_idx"]) if "layer_idx" in kwargs else self.layer_idx
    T = hidden_states.shape[1]
    Hq, Hkv = self.q_proj.weight.shape[0] // D, self.k_proj.weight.shape[0] // D
    x = hidden_states[0]
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    w_qkv = _fused_qkv_weight(self)
    if w_qkv is not None:
        qkv = ops.gemm_nt(x, w_qkv)
    else:  # three projections into column ranges of one buffer
        qkv = ops._empty((T, (Hq + 2 * Hkv) * D), dtype=torch.bfloat16, device=x.device)
        col = 0
        for proj in (self.q_proj, self.k_proj, self.v_proj):
            n = proj.weight.shape[0]
            w = proj.weight if proj.weight.stride(1) == 1 and proj.weight.stride(0) % 8 == 0 else proj.weight.contiguous()
            ops.gemm_nt(x, w, out=qkv[:, col:col + n])
            col += n
    q = ops._empty((T, Hq, D), dtype=torch.bfloat16, device=x.device)
    ops.qk_norm_rope_store(qkv, self.q_norm.weight, self.k_norm.weight, cos[0], sin[0], None, ctx.slot_mapping, q,
                           ctx.key_cache[layer_idx], ctx.value_cache[layer_idx], Hq, Hkv, D,
                           self.q_norm.variance_epsilon)
    # The kernel writes every row that belongs to a sequence with at least one key; what it leaves alone here are the
    # padding rows of a captured bucket, whose values nobody reads, so the output skips the NaN fill that
    # torch.empty adds under deterministic algorithms (one more launch per layer).
    k_cache, v_cache = ctx.key_cache[layer_idx], ctx.value_cache[layer_idx]
    if not (ctx.query_start_loc.dtype == ctx.context_lens.dtype == ctx.block_tables.dtype == torch.int32
            and ctx.query_start_loc.is_contiguous() and ctx.context_lens.is_contiguous() and ctx.block_tables.stride(-1) == 1
            and ctx.query_start_loc.is_cuda and ctx.context_lens.is_cuda and ctx.block_tables.is_cuda
            and k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.dtype == v_cache.dtype == torch.bfloat16):
        out, _ = flash_attn_varlen_func(
            q, k_cache, v_cache, cu_seqlens_q=ctx.query_start_loc, max_seqlen_q=ctx.max_seqlen_q,
            seqused_k=ctx.context_lens, page_table=ctx.block_tables, dropout_p=0.0, softmax_scale=self.scaling, causal=True)
    else:
        out = ops.paged_attention(q, k_cache, v_cache, ctx.query_start_loc, ctx.context_lens, ctx.block_tables,
                                  float(self.scaling), max_seqlen_q=int(ctx.max_seqlen_q or 0),
                                  out=ops._empty((T, Hq, v_cache.shape[-1]), dtype=torch.bfloat16, device=x.device))
    return self.o_proj(out.reshape(1, T, -1)), None


_ORIGINAL_LAYER = None  # Qwen3MoeDecoderLayer.forward while the fused form is patched in


def fused_decoder_layer_forward(self, hidden_states, attention_mask=None, position_ids=None, past_key_values=None,
                                use_cache=False, position_embeddings=None, **kwargs):
    """``Qwen3MoeDecoderLayer.forward`` with its two residual additions folded into the kernels next to them:
    ``residual + attention output`` into the post-attention RMSNorm's launch (which also writes the sum) and
    ``residual + MoE output`` into the MoE combine. Each sum is rounded to bf16 exactly where the separate
    addition rounds it, so the bits do not change. Taken under batch-invariant mode for bf16 GPU tensors without
    autograd when the layer's MLP is the patched sparse block; otherwise the original forward runs."""
    from transformers.models.qwen3_moe import modeling_qwen3_moe as hf

    from ...batch_invariant_ops import is_batch_invariant_mode_enabled

    norm = self.post_attention_layernorm
    if not (hidden_states.is_cuda and hidden_states.dtype == torch.bfloat16 and hidden_states.dim() == 3
            and not torch.is_grad_enabled() and is_batch_invariant_mode_enabled()
            and isinstance(self.mlp, hf.Qwen3MoeSparseMoeBlock) and isinstance(getattr(self.mlp, "experts", None), Qwen3MoeExperts)
            and hf.Qwen3MoeSparseMoeBlock.forward is moe_block_forward and norm.weight.dtype == torch.bfloat16):
        return _ORIGINAL_LAYER(self, hidden_states, attention_mask=attention_mask, position_ids=position_ids,
                               past_key_values=past_key_values, use_cache=use_cache,
                               position_embeddings=position_embeddings, **kwargs)
    residual = hidden_states if hidden_states.stride(2) == 1 else hidden_states.contiguous()
    attn_out, _ = self.self_attn(
        hidden_states=self.input_layernorm(hidden_states), attention_mask=attention_mask, position_ids=position_ids,
        past_key_values=past_key_values, use_cache=use_cache, position_embeddings=position_embeddings, **kwargs)
    summed = ops._empty_like(residual)
    normed = ops.rms_norm(attn_out, norm.weight, norm.variance_epsilon, hf_two_rounding=True, residual=residual,
                          sum_out=summed)
    return self.mlp(normed, residual=summed)


def apply_qwen3_moe_patches(fused_rms_norm: bool = True, fused_rope: bool = True, fused_attention: bool = True,
                            fused_residual: bool = True) -> None:
    """Swap the HuggingFace block's constructor and forward (idempotent). ``fused_rms_norm`` also replaces
    ``Qwen3MoeRMSNorm.forward`` by ``fused_rms_norm_forward`` (same bits under batch-invariant mode, one launch
    instead of eleven; not in the reference, whose optional Liger patch leaves RMSNorm alone because Liger's is
    not batch invariant, vexact/models/register.py:84-87) and ``fused_rope`` the modeling file's
    ``apply_rotary_pos_emb`` by ``fused_apply_rotary_pos_emb`` (the function that Liger patch swaps, :77-80).
    ``fused_attention`` replaces ``Qwen3MoeAttention.forward`` by ``fused_attention_forward`` (same bits; it
    applies to steps over the paged cache and falls through to the original otherwise) and ``fused_residual``
    ``Qwen3MoeDecoderLayer.forward`` by ``fused_decoder_layer_forward`` (same bits, two launches fewer)."""
    global _ORIGINAL, _ORIGINAL_NORM, _ORIGINAL_ROPE, _ORIGINAL_ATTN, _ORIGINAL_LAYER
    from transformers.models.qwen3_moe import modeling_qwen3_moe as hf

    if _ORIGINAL is None:
        _ORIGINAL = (hf.Qwen3MoeSparseMoeBlock.__init__, hf.Qwen3MoeSparseMoeBlock.forward)
        hf.Qwen3MoeSparseMoeBlock.__init__ = moe_block_init
        hf.Qwen3MoeSparseMoeBlock.forward = moe_block_forward
    if fused_rms_norm and _ORIGINAL_NORM is None:
        _ORIGINAL_NORM = hf.Qwen3MoeRMSNorm.forward
        hf.Qwen3MoeRMSNorm.forward = fused_rms_norm_forward
    if fused_rope and _ORIGINAL_ROPE is None:
        _ORIGINAL_ROPE = hf.apply_rotary_pos_emb
        hf.apply_rotary_pos_emb = fused_apply_rotary_pos_emb
    if fused_attention and _ORIGINAL_ATTN is None:
        _ORIGINAL_ATTN = hf.Qwen3MoeAttention.forward
        hf.Qwen3MoeAttention.forward = fused_attention_forward
    if fused_residual and _ORIGINAL_LAYER is None:
        _ORIGINAL_LAYER = hf.Qwen3MoeDecoderLayer.forward
        hf.Qwen3MoeDecoderLayer.forward = fused_decoder_layer_forward


def remove_qwen3_moe_patches() -> None:
    """Put the HuggingFace block's own constructor and forward back (blocks built meanwhile keep their fused
    experts and stop working with the original forward; meant for tests and tools that need both forms)."""
    global _ORIGINAL, _ORIGINAL_NORM, _ORIGINAL_ROPE, _ORIGINAL_ATTN, _ORIGINAL_LAYER
    from transformers.models.qwen3_moe import modeling_qwen3_moe as hf

    if _ORIGINAL_LAYER is not None:
        hf.Qwen3MoeDecoderLayer.forward = _ORIGINAL_LAYER
        _ORIGINAL_LAYER = None
    if _ORIGINAL_ATTN is not None:
        hf.Qwen3MoeAttention.forward = _ORIGINAL_ATTN
        _ORIGINAL_ATTN = None
    if _ORIGINAL_ROPE is not None:
        hf.apply_rotary_pos_emb = _ORIGINAL_ROPE
        _ORIGINAL_ROPE = None
    if _ORIGINAL is not None:
        hf.Qwen3MoeSparseMoeBlock.__init__, hf.Qwen3MoeSparseMoeBlock.forward = _ORIGINAL
        _ORIGINAL = None
    if _ORIGINAL_NORM is not None:
        hf.Qwen3MoeRMSNorm.forward = _ORIGINAL_NORM
        _ORIGINAL_NORM = None
