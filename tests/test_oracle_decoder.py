"""Pins the decoder oracle (oracle/decoder.py) against HuggingFace's own CPU routines for the layer the
reference patches: rotary tables and rotation bit for bit, the per-head norm + rotary + cache-write glue
against the module's own q_norm / k_norm / apply_rotary_pos_emb, one decoder layer and a whole
prefill + decode step against ``Qwen3MoeDecoderLayer`` / ``Qwen3MoeForCausalLM`` (eager attention, eager
experts). Norm weights are far from 1 and differ between q and k, so a swapped weight, a weight applied at
the wrong rounding point, a wrong rope_theta or half layout fails here."""

import types

import numpy as np
import pytest
import torch

from oracle import decoder as OD
from oracle.metadata import prepare_gen_ctx_ref

hf = pytest.importorskip("transformers.models.qwen3_moe.modeling_qwen3_moe")
from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig  # noqa: E402

BF = torch.bfloat16


def _hf_config(layers=2, theta=1.0e6, max_pos=4096):
    return Qwen3MoeConfig(
        vocab_size=160, hidden_size=64, intermediate_size=96, num_hidden_layers=layers, num_attention_heads=4,
        num_key_value_heads=2, head_dim=32, num_experts=8, num_experts_per_tok=2, moe_intermediate_size=32,
        norm_topk_prob=True, max_position_embeddings=max_pos, rms_norm_eps=1e-6,
        rope_parameters={"rope_type": "default", "rope_theta": theta}, attn_implementation="eager")


def _oracle_cfg(c):
    return types.SimpleNamespace(
        hidden_size=c.hidden_size, num_layers=c.num_hidden_layers, num_heads=c.num_attention_heads,
        num_kv_heads=c.num_key_value_heads, head_dim=c.head_dim, num_experts=c.num_experts, top_k=c.num_experts_per_tok,
        moe_intermediate=c.moe_intermediate_size, vocab_size=c.vocab_size, rms_eps=c.rms_norm_eps,
        norm_topk_prob=c.norm_topk_prob, page_size=4)


def _randomise(model, seed):
    """bf16 weights ~ N(0, 0.08); norm weights uniform in [0.5, 1.5], all different."""
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if "norm" in name:
                p.copy_(0.5 + torch.rand(p.shape, generator=g))
            else:
                p.copy_(0.08 * torch.randn(p.shape, generator=g))
    for p in model.parameters():  # parameters only: a rotary embedding's inv_freq buffer stays fp32
        p.data = p.data.to(BF)
    return model.eval()


def _layer_weights(layer):
    a, m = layer.self_attn, layer.mlp
    return dict(
        in_norm=layer.input_layernorm.weight.data, post_norm=layer.post_attention_layernorm.weight.data,
        qkv=torch.cat([a.q_proj.weight.data, a.k_proj.weight.data, a.v_proj.weight.data], dim=0),
        q_norm=a.q_norm.weight.data, k_norm=a.k_norm.weight.data, o=a.o_proj.weight.data,
        router=m.gate.weight.data, gate_up=m.experts.gate_up_proj.data, down=m.experts.down_proj.data)


def _causal_mask(n):
    return torch.full((n, n), float("-inf")).triu(1)[None, None].to(BF)


def _record_routing(layers):
    """Forward hooks that keep every layer's expert choice, so that the oracle can be put on the same
    experts at near-ties."""
    log, handles = [], []
    for l in layers:
        handles.append(l.mlp.gate.register_forward_hook(lambda mod, args, out: log.append(out[2].clone())))
    return log, handles


def test_rope_tables_equal_huggingface_rotary_embedding_bitwise():
    for theta, D in ((1.0e6, 128), (1.0e4, 64), (5.0e5, 32)):
        c = _hf_config(theta=theta, max_pos=40960)
        c.head_dim = D
        rot = hf.Qwen3MoeRotaryEmbedding(c)
        pos = torch.cat([torch.arange(0, 300), torch.arange(4000, 4100), torch.arange(40900, 40960)])
        cos_hf, sin_hf = rot(torch.zeros(1, 1, dtype=BF), pos[None])
        cos, sin = OD.rope_tables_ref(D, theta, 40960)
        assert torch.equal(cos[pos].view(torch.int16), cos_hf[0].view(torch.int16))
        assert torch.equal(sin[pos].view(torch.int16), sin_hf[0].view(torch.int16))
    # closed forms: position 0 is the identity rotation; the first pair turns by exactly `position` radians
    cos, sin = OD.rope_tables_ref(128, 1.0e6, 16)
    assert bool((cos[0] == 1).all()) and bool((sin[0] == 0).all())
    assert torch.equal(cos[:, 0], torch.arange(16.0).cos().to(BF)) and torch.equal(sin[:, 64], torch.arange(16.0).sin().to(BF))


def test_rope_ref_equals_huggingface_apply_rotary_pos_emb_bitwise():
    g = torch.Generator().manual_seed(11)
    T, Hq, Hkv, D = 37, 6, 2, 128
    q = torch.randn(T, Hq, D, generator=g).to(BF)
    k = torch.randn(T, Hkv, D, generator=g).to(BF)
    cos_t, sin_t = OD.rope_tables_ref(D, 1.0e6, 40960)
    pos = torch.randint(0, 40960, (T,), generator=g)
    cos, sin = cos_t[pos], sin_t[pos]
    q_hf, k_hf = hf.apply_rotary_pos_emb(q.transpose(0, 1)[None], k.transpose(0, 1)[None], cos[None], sin[None])
    assert torch.equal(OD.rope_ref(q, cos, sin).view(torch.int16), q_hf[0].transpose(0, 1).contiguous().view(torch.int16))
    assert torch.equal(OD.rope_ref(k, cos, sin).view(torch.int16), k_hf[0].transpose(0, 1).contiguous().view(torch.int16))
    # a rotation keeps each (j, j + D/2) pair's length up to bf16 rounding, and a wrong half layout
    # (interleaved pairs) would not
    r = OD.rope_ref(q, cos, sin).float()
    n0 = q.float()[..., : D // 2] ** 2 + q.float()[..., D // 2:] ** 2
    n1 = r[..., : D // 2] ** 2 + r[..., D // 2:] ** 2
    assert float((n1 - n0).abs().max()) <= 0.05 * float(n0.max())


def test_qk_norm_rope_store_ref_equals_huggingface_attention_front_end():
    c = _hf_config()
    attn = _randomise(hf.Qwen3MoeAttention(c, 0), 5)
    Hq, Hkv, D = c.num_attention_heads, c.num_key_value_heads, c.head_dim
    g = torch.Generator().manual_seed(6)
    T = 11
    qkv = torch.randn(T, (Hq + 2 * Hkv) * D, generator=g).to(BF)
    pos = torch.tensor([0, 1, 2, 3, 4, 4095, 17, 18, 19, 20, 21])
    slots = torch.tensor([8, 9, 10, 11, 0, 1, -1, 2, 3, 20, 21], dtype=torch.int32)
    cos_t, sin_t = OD.rope_tables_ref(D, 1.0e6, 4096)
    kc, vc = torch.zeros(6, 4, Hkv, D, dtype=BF), torch.zeros(6, 4, Hkv, D, dtype=BF)
    q, k = OD.qk_norm_rope_store_ref(qkv, attn.q_norm.weight.data, attn.k_norm.weight.data, cos_t, sin_t, pos, slots,
                                     kc, vc, Hq, Hkv, D)
    # the module's own norm layers and rotation on the same split
    with torch.no_grad():
        q_hf = attn.q_norm(qkv[:, : Hq * D].view(1, T, Hq, D)).transpose(1, 2)
        k_hf = attn.k_norm(qkv[:, Hq * D: (Hq + Hkv) * D].view(1, T, Hkv, D)).transpose(1, 2)
        q_hf, k_hf = hf.apply_rotary_pos_emb(q_hf, k_hf, cos_t[pos][None], sin_t[pos][None])
    assert torch.equal(q, q_hf[0].transpose(0, 1)) and torch.equal(k, k_hf[0].transpose(0, 1))
    v = qkv[:, (Hq + Hkv) * D:].view(T, Hkv, D)
    flat_k, flat_v = kc.view(-1, Hkv, D), vc.view(-1, Hkv, D)
    written = set()
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        written.add(s)
        assert torch.equal(flat_k[s], k[t]) and torch.equal(flat_v[s], v[t])
    rest = [s for s in range(flat_k.shape[0]) if s not in written]
    assert bool((flat_k[rest] == 0).all()) and bool((flat_v[rest] == 0).all())
    # q and k norm weights are really different tensors in this test
    assert not torch.equal(attn.q_norm.weight.data, attn.k_norm.weight.data)


def _paged_request_meta(lens, new, page):
    pages = [-(-n // page) for n in lens]
    perm = np.random.default_rng(0).permutation(sum(pages) + 3)
    blocks, o = [], 0
    for p in pages:
        blocks.append(perm[o: o + p].tolist())
        o += p
    reqs = [dict(num_computed_tokens=n, tokens_this_step=t, block_ids=b) for n, t, b in zip(lens, new, blocks)]
    return prepare_gen_ctx_ref(reqs, page, max(pages) + 1), len(perm)


def test_layer_ref_against_huggingface_decoder_layer():
    c = _hf_config()
    cfg = _oracle_cfg(c)
    layer = _randomise(hf.Qwen3MoeDecoderLayer(c, 0), 21)
    lw = _layer_weights(layer)
    rot = hf.Qwen3MoeRotaryEmbedding(c)
    cos_t, sin_t = OD.rope_tables_ref(c.head_dim, 1.0e6, 4096)
    g = torch.Generator().manual_seed(22)
    lens = [13, 6]
    xs = [torch.randn(n, c.hidden_size, generator=g).to(BF) for n in lens]
    # HuggingFace: each sequence alone under a causal mask; its expert choice recorded
    log, handles = _record_routing([layer])
    want = []
    with torch.no_grad():
        for x in xs:
            n = x.shape[0]
            pe = rot(x[None], torch.arange(n)[None])
            want.append(layer(x[None], attention_mask=_causal_mask(n), position_embeddings=pe)[0])
    for h in handles:
        h.remove()
    want = torch.cat(want)
    # oracle: both sequences in one packed step through a paged cache
    meta, nblocks = _paged_request_meta(lens, lens, cfg.page_size)
    kc = torch.zeros(nblocks, cfg.page_size, cfg.num_kv_heads, cfg.head_dim, dtype=BF)
    vc = torch.zeros_like(kc)
    report = []
    got = OD.layer_ref(cfg, lw, torch.cat(xs), torch.as_tensor(meta["positions"]), meta, kc, vc, cos_t, sin_t,
                       forced_idx=torch.cat(log), report=report)
    assert sum(r["differ"] for r in report) <= 2, report  # own routing agrees except at near-ties
    # fused-order experts and fp32-score attention against HuggingFace's bf16 eager forms: bf16-level agreement
    err = (got.float() - want.float()).abs()
    scale = float(want.float().abs().max())
    # (measured 0.8 % / 0.03 % of the largest entry; q and k norm weights swapped: 4.3 % / 0.6 %)
    assert float(err.max()) <= 2e-2 * scale, (float(err.max()), scale)
    assert float(err.mean()) <= 1e-3 * scale
    # the same layer in fp32 (weights still the bf16 values) as a second, rounding-free reference
    layer32 = hf.Qwen3MoeDecoderLayer(c, 0).eval()
    layer32.load_state_dict({k_: v_.float() for k_, v_ in layer.state_dict().items()})
    want32 = []
    with torch.no_grad():
        for x in xs:
            n = x.shape[0]
            pe = hf.Qwen3MoeRotaryEmbedding(c)(x[None].float(), torch.arange(n)[None])
            want32.append(layer32(x[None].float(), attention_mask=_causal_mask(n).float(), position_embeddings=pe)[0])
    want32 = torch.cat(want32)
    routed_same = torch.cat(log).sort(-1).values  # fp32 routing may differ at near-ties: compare where it agrees
    err32 = (got.float() - want32).abs().max(-1).values
    assert float(err32.median()) <= 3e-2 * float(want32.abs().max())
    assert routed_same.shape[0] == sum(lens)


def test_decoder_step_ref_prefill_and_decode_against_huggingface_causal_lm():
    c = _hf_config(layers=2)
    cfg = _oracle_cfg(c)
    model = _randomise(hf.Qwen3MoeForCausalLM(c), 31)
    weights = types.SimpleNamespace(
        embed=model.model.embed_tokens.weight.data, lm_head=model.lm_head.weight.data,
        final_norm=model.model.norm.weight.data, layers=[_layer_weights(l) for l in model.model.layers])
    cos_t, sin_t = OD.rope_tables_ref(c.head_dim, 1.0e6, 4096)
    rng = np.random.default_rng(32)
    lens = [9, 14, 5]
    prompts = [rng.integers(0, c.vocab_size, size=n + 1) for n in lens]  # the last id is the decode step's input

    def hf_last_logits(ids):
        log, handles = _record_routing(model.model.layers)
        with torch.no_grad():
            out = model(input_ids=torch.as_tensor(ids)[None]).logits[0, -1]
        for h in handles:
            h.remove()
        return out, log

    # prefill of the first n tokens of every prompt in one packed step
    meta, nblocks = _paged_request_meta([n + 1 for n in lens], [n + 1 for n in lens], cfg.page_size)
    blocks = [[int(b) for b in row if b >= 0] for row in meta["block_tables"]]
    reqs = [dict(num_computed_tokens=n, tokens_this_step=n, block_ids=b) for n, b in zip(lens, blocks)]
    pmeta = prepare_gen_ctx_ref(reqs, cfg.page_size, meta["block_tables"].shape[1])
    kc = [torch.zeros(nblocks, cfg.page_size, cfg.num_kv_heads, cfg.head_dim, dtype=BF) for _ in range(2)]
    vc = [torch.zeros_like(t) for t in kc]
    hf_pre = [hf_last_logits(p[:n]) for p, n in zip(prompts, lens)]
    forced = [torch.cat([log[li] for _, log in hf_pre]) for li in range(2)]
    report = []
    logits, _, _ = OD.decoder_step_ref(cfg, weights, np.concatenate([p[:n] for p, n in zip(prompts, lens)]), pmeta, kc, vc,
                                       cos_t, sin_t, forced, report)
    want = torch.stack([l for l, _ in hf_pre])
    assert sum(r["differ"] for r in report) <= 0.1 * sum(r["tokens"] for r in report)
    lp, lp_want = torch.log_softmax(logits.float(), -1), torch.log_softmax(want.float(), -1)
    assert float((lp - lp_want).abs().max()) <= 5e-2, float((lp - lp_want).abs().max())
    assert float((logits.float() - want.float()).abs().max()) <= 3e-2 * float(want.float().abs().max())

    # one decode step on top of the caches the prefill wrote; HuggingFace recomputes the whole sequence
    dreqs = [dict(num_computed_tokens=n + 1, tokens_this_step=1, block_ids=b) for n, b in zip(lens, blocks)]
    dmeta = prepare_gen_ctx_ref(dreqs, cfg.page_size, meta["block_tables"].shape[1])
    hf_dec = [hf_last_logits(p) for p in prompts]
    forced = [torch.stack([log[li][-1] for _, log in hf_dec]) for li in range(2)]
    report = []
    logits, tokens, logprobs = OD.decoder_step_ref(cfg, weights, np.array([p[-1] for p in prompts]), dmeta, kc, vc,
                                                   cos_t, sin_t, forced, report)
    want = torch.stack([l for l, _ in hf_dec])
    lp, lp_want = torch.log_softmax(logits.float(), -1), torch.log_softmax(want.float(), -1)
    assert float((lp - lp_want).abs().max()) <= 5e-2, float((lp - lp_want).abs().max())
    # the step's own outputs: greedy token and its log-probability
    assert torch.equal(tokens, logits.float().argmax(-1))
    assert torch.allclose(logprobs, lp.gather(-1, tokens[:, None])[:, 0], atol=1e-6)
    # a model with the wrong rope_theta is NOT within that tolerance (the test has teeth)
    bad_cos, bad_sin = OD.rope_tables_ref(c.head_dim, 1.0e4, 4096)
    kc2 = [torch.zeros_like(t) for t in kc]
    vc2 = [torch.zeros_like(t) for t in vc]
    bad, _, _ = OD.decoder_step_ref(cfg, weights, np.concatenate([p[:n] for p, n in zip(prompts, lens)]), pmeta, kc2, vc2,
                                    bad_cos, bad_sin, None, None)
    good_ref = torch.stack([l for l, _ in hf_pre])
    assert float((bad.float() - good_ref.float()).abs().max()) > 3e-2 * float(good_ref.float().abs().max())
