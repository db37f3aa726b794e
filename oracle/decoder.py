"""Oracle (test infrastructure): a Qwen3-MoE-shaped decoder step on the CPU, composed from the
other oracle functions. Follows the HuggingFace Qwen3-MoE layer the reference patches
(call order summarised in vexact/models/qwen3_moe/modeling_qwen3_moe.py:119-145 for the MoE block and
vexact/batch_invariant_ops/triton_invariant_attention.py:1047-1070 for cache write + attention)."""

from __future__ import annotations

import torch

from .attention import eager_attention, gather_paged, store_kvcache_ref
from .moe import fused_moe_ref, router_ref, router_weights_for
from .row_ops import hf_rms_norm_ref, logprobs_ref, matmul_ref


def _bf(x):
    return x.to(torch.bfloat16)


def rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def rope_tables_ref(head_dim: int, rope_theta: float, max_positions: int):
    """cos / sin ``[max_positions, D]`` in bf16 from ``rope_theta`` alone: ``inv_freq = theta^(-2i/D)``
    (fp32), ``angle = position * inv_freq`` (one fp32 product), the ``D/2`` angles repeated over both
    halves, cos / sin in fp32, then cast: HuggingFace's default rotary embedding for bf16 activations,
    the un-overridden glue of the layer the reference patches
    (vexact/models/qwen3_moe/modeling_qwen3_moe.py:119-145 runs inside that layer)."""
    inv_freq = 1.0 / (rope_theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    angle = torch.arange(max_positions, dtype=torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat((angle, angle), dim=-1)
    return _bf(emb.cos()), _bf(emb.sin())


def rope_ref(x, cos, sin):
    """``x * cos + rotate_half(x) * sin`` in bf16 tensor ops; ``x [T,H,D]``, ``cos/sin [T,D]``."""
    c, s = cos.unsqueeze(1), sin.unsqueeze(1)
    return _bf(_bf(x.float() * c.float()).float() + _bf(rotate_half(x).float() * s.float()).float())


def embedding_ref(table, ids):
    """Row gather ``table[ids]``."""
    return table[torch.as_tensor(ids).long()]


def qk_norm_rope_store_ref(qkv, q_norm_w, k_norm_w, cos_t, sin_t, positions, slot_mapping, k_cache, v_cache,
                           num_heads: int, num_kv_heads: int, head_dim: int, eps: float = 1e-6):
    """What sits between the q/k/v projection and attention in the patched layer: split the fused
    projection ``[T, (Hq+2Hkv) D]``, per-head RMSNorm of q and k (HuggingFace's two-rounding form, each with
    its OWN weight), rotary embedding at ``positions``, and the cache write of k and v at
    ``slot_mapping`` (vexact/batch_invariant_ops/triton_invariant_attention.py:1047-1054 with
    vexact/batch_invariant_ops/kv_cache_context.py:294-314). Caches are written in place (``None``: no
    write); returns (q, k) after the rotary embedding."""
    T = qkv.shape[0]
    Hq, Hkv, D = num_heads, num_kv_heads, head_dim
    q = qkv[:, : Hq * D].reshape(T, Hq, D)
    k = qkv[:, Hq * D : (Hq + Hkv) * D].reshape(T, Hkv, D)
    v = qkv[:, (Hq + Hkv) * D :].reshape(T, Hkv, D)
    q = hf_rms_norm_ref(q, q_norm_w, eps)
    k = hf_rms_norm_ref(k, k_norm_w, eps)
    pos = torch.as_tensor(positions).long()
    cos, sin = cos_t[pos], sin_t[pos]
    q, k = rope_ref(q, cos, sin), rope_ref(k, cos, sin)
    if k_cache is not None:
        store_kvcache_ref(k, v.contiguous(), k_cache, v_cache, slot_mapping)
    return q, k


def layer_ref(cfg, lw, x, positions, meta, k_cache, v_cache, cos_t, sin_t, forced_idx=None, report=None):
    """One decoder layer on ``x [T,H]`` (bf16); writes this step's K/V into the caches.

    ``forced_idx [T,k]``: expert choice of another implementation. Two implementations whose router
    logits differ by a bf16 ulp pick different experts at near-ties, after which hidden states are
    not comparable; the oracle then follows the forced choice, and records in ``report`` how many
    tokens differed from its own choice and the largest logit gap it had to cross to do so."""
    T = x.shape[0]
    Hq, Hkv, D, I = cfg.num_heads, cfg.num_kv_heads, cfg.head_dim, cfg.moe_intermediate
    h = hf_rms_norm_ref(x, lw["in_norm"], cfg.rms_eps)
    qkv = matmul_ref(h, lw["qkv"].t())
    q, _ = qk_norm_rope_store_ref(qkv, lw["q_norm"], lw["k_norm"], cos_t, sin_t, positions, meta["slot_mapping"],
                                  k_cache, v_cache, Hq, Hkv, D, cfg.rms_eps)
    outs = []
    qsl, lens, bt = meta["query_start_loc"], meta["context_lens"], meta["block_tables"]
    for s in range(len(lens)):
        q0, q1, n = int(qsl[s]), int(qsl[s + 1]), int(lens[s])
        if q1 <= q0:
            continue
        ks = gather_paged(k_cache, torch.as_tensor(bt[s]), n)
        vs = gather_paged(v_cache, torch.as_tensor(bt[s]), n)
        outs.append(eager_attention(q[q0:q1], ks, vs, D ** -0.5))
    attn = torch.cat(outs, dim=0).reshape(T, Hq * D)
    x = _bf(x.float() + matmul_ref(attn, lw["o"].t()).float())
    h2 = hf_rms_norm_ref(x, lw["post_norm"], cfg.rms_eps)
    logits = matmul_ref(h2, lw["router"].t())
    w, idx = router_ref(logits, cfg.top_k, renorm=cfg.norm_topk_prob)
    if forced_idx is not None:
        f = forced_idx.to(torch.int64)
        differs = (f.sort(-1).values != idx.sort(-1).values).any(-1)
        if report is not None:
            lf = logits.float()
            kth = lf.gather(-1, idx)[:, -1:]  # own k-th best logit
            gap = (kth - lf.gather(-1, f)).clamp_(min=0).max(-1).values  # how far below it the forced picks lie
            report.append({"tokens": int(differs.numel()), "differ": int(differs.sum()),
                           "max_gap": float(gap[differs].max()) if bool(differs.any()) else 0.0,
                           "max_gap_rel": float((gap / kth.abs().clamp_(min=1e-3).squeeze(-1))[differs].max()) if bool(differs.any()) else 0.0})
        idx = f
        w = router_weights_for(logits, idx, renorm=cfg.norm_topk_prob)
    gu = lw["gate_up"]
    m = fused_moe_ref(h2, w, idx, gu[:, :I, :], gu[:, I:, :], lw["down"])
    return _bf(x.float() + m.float())


def decoder_step_ref(cfg, weights, input_ids, meta, key_cache, value_cache, cos_t, sin_t, forced_routing=None,
                     report=None):
    """Full step: embedding, all layers, final norm, lm_head on each sequence's last token, greedy
    token and its fp32 logprob (vexact/inferencer/inferencer.py:391-449)."""
    x = embedding_ref(weights.embed, input_ids)
    pos = torch.as_tensor(meta["positions"]).long()
    for li, lw in enumerate(weights.layers):
        forced = forced_routing[li] if forced_routing is not None else None
        x = layer_ref(cfg, lw, x, pos, meta, key_cache[li], value_cache[li], cos_t, sin_t, forced, report)
    h = hf_rms_norm_ref(x, weights.final_norm, cfg.rms_eps)
    last = torch.as_tensor(meta["query_start_loc"][1:]).long() - 1
    logits = matmul_ref(h[last], weights.lm_head.t())
    tokens = logits.float().argmax(dim=-1)
    return logits, tokens, logprobs_ref(logits.float(), tokens)
