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


def rope_ref(x, cos, sin):
    """``x * cos + rotate_half(x) * sin`` in bf16 tensor ops; ``x [T,H,D]``, ``cos/sin [T,D]``."""
    c, s = cos.unsqueeze(1), sin.unsqueeze(1)
    return _bf(_bf(x.float() * c.float()).float() + _bf(rotate_half(x).float() * s.float()).float())


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
    q = qkv[:, : Hq * D].reshape(T, Hq, D)
    k = qkv[:, Hq * D : (Hq + Hkv) * D].reshape(T, Hkv, D)
    v = qkv[:, (Hq + Hkv) * D :].reshape(T, Hkv, D)
    q = hf_rms_norm_ref(q, lw["q_norm"], cfg.rms_eps)
    k = hf_rms_norm_ref(k, lw["k_norm"], cfg.rms_eps)
    cos, sin = cos_t[positions], sin_t[positions]
    q, k = rope_ref(q, cos, sin), rope_ref(k, cos, sin)
    store_kvcache_ref(k, v.contiguous(), k_cache, v_cache, meta["slot_mapping"])
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
    x = weights.embed[torch.as_tensor(input_ids).long()]
    pos = torch.as_tensor(meta["positions"]).long()
    for li, lw in enumerate(weights.layers):
        forced = forced_routing[li] if forced_routing is not None else None
        x = layer_ref(cfg, lw, x, pos, meta, key_cache[li], value_cache[li], cos_t, sin_t, forced, report)
    h = hf_rms_norm_ref(x, weights.final_norm, cfg.rms_eps)
    last = torch.as_tensor(meta["query_start_loc"][1:]).long() - 1
    logits = matmul_ref(h[last], weights.lm_head.t())
    tokens = logits.float().argmax(dim=-1)
    return logits, tokens, logprobs_ref(logits.float(), tokens)
