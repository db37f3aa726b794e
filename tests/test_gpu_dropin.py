"""The drop-in seen from the reference's callers: a HuggingFace ``Qwen3MoeForCausalLM`` driven the way
``Inferencer`` drives it (vexact/inferencer/inferencer.py:52-55, 124-191, 351-383; model wrapper
vexact/inferencer/model_loader.py:217-278): the attention function registered under the reference's name
in ``ALL_ATTENTION_FUNCTIONS``, the MoE block patched, batch-invariant mode on, a thread-local paged KV
context per step, packed batch of size 1. Paged prefill of three prompts, then a decode step: every
request alone gives the bits it gives in the batch, and the logprobs agree with the CPU oracle of the
whole decoder (the assertions of tests/test_inferencer.py:300-595 without the stored tensors of a real
checkpoint)."""

import types

import numpy as np
import pytest
import torch

from oracle import decoder as OD
from tests.util import assert_bitwise

pytestmark = pytest.mark.gpu

BF = torch.bfloat16


def _build_model(seed):
    from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeForCausalLM

    cfg = Qwen3MoeConfig(
        vocab_size=1000, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
        num_key_value_heads=2, head_dim=128, num_experts=8, num_experts_per_tok=2, moe_intermediate_size=128,
        norm_topk_prob=True, max_position_embeddings=512, rms_norm_eps=1e-6,
        rope_parameters={"rope_type": "default", "rope_theta": 1.0e6})
    cfg._attn_implementation = "triton-invariant"
    model = Qwen3MoeForCausalLM(cfg)
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if "norm" in name:
                p.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=g))
            else:
                p.copy_(0.05 * torch.randn(p.shape, generator=g))
    for p in model.parameters():  # parameters only: the rotary embedding's inv_freq buffer stays fp32, as in a
        p.data = p.data.to(BF)    # model created by the reference's loader (model_loader.py:307-320)
    return cfg, model.eval()


def _oracle_weights(model):
    layers = []
    for l in model.model.layers:
        a, m = l.self_attn, l.mlp
        layers.append({k: v.detach().cpu() for k, v in dict(
            in_norm=l.input_layernorm.weight, post_norm=l.post_attention_layernorm.weight,
            qkv=torch.cat([a.q_proj.weight, a.k_proj.weight, a.v_proj.weight], dim=0), q_norm=a.q_norm.weight,
            k_norm=a.k_norm.weight, o=a.o_proj.weight, router=m.gate.weight, gate_up=m.experts.gate_up_proj,
            down=m.experts.down_proj).items()})
    return types.SimpleNamespace(embed=model.model.embed_tokens.weight.detach().cpu(), lm_head=model.lm_head.weight.detach().cpu(),
                                 final_norm=model.model.norm.weight.detach().cpu(), layers=layers)


def test_huggingface_causal_lm_through_the_registered_interfaces():
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    from vexact_amd.batch_invariant_ops import flash_attention_forward, set_batch_invariant_mode
    from vexact_amd.batch_invariant_ops.standalone_logprobs import logprobs_from_logits_flash_attn
    from vexact_amd.batch_invariant_ops.kv_cache_context import (KVCacheManager, KVCacheStore, clear_kv_cache_context,
                                                                 set_kv_cache_context)
    from vexact_amd.decoder import build_step_metadata
    from vexact_amd.models.qwen3_moe import apply_qwen3_moe_patches, remove_qwen3_moe_patches

    page, max_blocks_per_req = 16, 32
    cache_cfg = types.SimpleNamespace(page_size=page, max_cache_blocks=64)
    had = ALL_ATTENTION_FUNCTIONS._global_mapping.get("triton-invariant") if hasattr(ALL_ATTENTION_FUNCTIONS, "_global_mapping") else None
    ALL_ATTENTION_FUNCTIONS["triton-invariant"] = flash_attention_forward
    apply_qwen3_moe_patches()
    try:
        hf_cfg, model = _build_model(seed=17)
        model = model.cuda()
        weights = _oracle_weights(model)
        store = KVCacheStore(hf_cfg, cache_cfg, torch.device("cuda"))
        alloc = KVCacheManager(cache_cfg)
        rng = np.random.default_rng(18)
        lens = [37, 5, 120]
        prompts = [rng.integers(0, hf_cfg.vocab_size, size=n) for n in lens]
        # blocks for prompt + one generated token, taken in turns so that the tables interleave
        blocks = [[] for _ in lens]
        for step in range(max(-(-(n + 1) // page) for n in lens)):
            for s, n in enumerate(lens):
                if step < -(-(n + 1) // page):
                    blocks[s] += list(alloc.allocate_blocks((step + 1) * page, step))
        routing = []
        hooks = [l.mlp.experts.register_forward_pre_hook(lambda mod, args, kw: routing.append(kw["selected_experts"].clone()),
                                                         with_kwargs=True) for l in model.model.layers]

        def step(which, new_tokens, ids):
            """One Inferencer step over the requests ``which``: returns (last-token logits, greedy tokens, logprobs, meta)."""
            reqs = [dict(num_computed_tokens=done, tokens_this_step=new, block_ids=blocks[s])
                    for s, (done, new) in zip(which, new_tokens)]
            meta = build_step_metadata(reqs, page, max_blocks_per_req)
            dev = {k: torch.as_tensor(v).cuda() for k, v in meta.items() if k != "max_seqlen_q"}
            set_kv_cache_context(is_paged_attn=True, key_cache=store.key_cache, value_cache=store.value_cache,
                                 block_tables=dev["block_tables"], context_lens=dev["context_lens"],
                                 slot_mapping=dev["slot_mapping"], query_start_loc=dev["query_start_loc"],
                                 max_seqlen_q=int(meta["max_seqlen_q"]))
            routing.clear()
            try:
                with torch.inference_mode(), set_batch_invariant_mode(True):
                    out = model.model(input_ids=torch.as_tensor(ids)[None].cuda(), position_ids=dev["positions"][None],
                                      use_cache=False, return_dict=True)
                    last = (dev["query_start_loc"][1:] - 1).long()
                    logits = model.lm_head(out.last_hidden_state)[0, last, :]
                    tokens = logits.argmax(-1)
                    lp = logprobs_from_logits_flash_attn(logits.float(), tokens)
            finally:
                clear_kv_cache_context()
            return logits.cpu(), tokens.cpu(), lp.cpu(), meta, [r.cpu() for r in routing]

        everyone = [0, 1, 2]
        # ---- paged prefill of the three prompts in one packed batch, then each alone
        logits_b, tok_b, lp_b, pmeta, prouting = step(everyone, [(n, n) for n in lens], np.concatenate(prompts))
        k_after_batch = store.key_cache[0].clone()
        for s in everyone:
            logits_1, tok_1, lp_1, _, _ = step([s], [(lens[s], lens[s])], prompts[s])
            assert_bitwise(logits_1, logits_b[s: s + 1], f"prefill logits of request {s}: alone vs in the batch")
            assert_bitwise(lp_1, lp_b[s: s + 1], f"prefill logprob of request {s}")
        assert_bitwise(store.key_cache[0], k_after_batch, "the cache holds the same keys either way")
        # ---- one decode step on top: batch vs alone
        dlogits_b, dtok_b, dlp_b, dmeta, drouting = step(everyone, [(n + 1, 1) for n in lens], tok_b.numpy())
        for s in everyone:
            dlogits_1, dtok_1, dlp_1, _, _ = step([s], [(lens[s] + 1, 1)], tok_b.numpy()[s: s + 1])
            assert_bitwise(dlogits_1, dlogits_b[s: s + 1], f"decode logits of request {s}: alone vs in the batch")
            assert_bitwise(dlp_1, dlp_b[s: s + 1], f"decode logprob of request {s}")
            assert int(dtok_1[0]) == int(dtok_b[s])
        for h in hooks:
            h.remove()

        # ---- the CPU oracle of the whole decoder on the same weights, following the GPU's expert choice at near-ties
        ocfg = types.SimpleNamespace(num_heads=4, num_kv_heads=2, head_dim=128, moe_intermediate=128, rms_eps=1e-6, top_k=2,
                                     norm_topk_prob=True)
        cos, sin = OD.rope_tables_ref(128, 1.0e6, 512)
        kc = [torch.zeros(64, page, 2, 128, dtype=BF) for _ in range(2)]
        vc = [torch.zeros_like(t) for t in kc]
        report = []
        ref_logits, _, _ = OD.decoder_step_ref(ocfg, weights, np.concatenate(prompts), pmeta, kc, vc, cos, sin, prouting, report)
        lp_ref = torch.log_softmax(ref_logits.float(), -1).gather(-1, tok_b[:, None])[:, 0]
        assert float((lp_b - lp_ref).abs().max()) <= 2e-2, "prefill logprob vs the decoder oracle"
        ref_logits, _, _ = OD.decoder_step_ref(ocfg, weights, tok_b.numpy(), dmeta, kc, vc, cos, sin, drouting, report)
        lp_ref = torch.log_softmax(ref_logits.float(), -1).gather(-1, dtok_b[:, None])[:, 0]
        assert float((dlp_b - lp_ref).abs().max()) <= 2e-2, "decode logprob vs the decoder oracle"
        differ, total = sum(r["differ"] for r in report), sum(r["tokens"] for r in report)
        assert differ <= 0.1 * total, f"routing differs on {differ} of {total} (token, layer) pairs"
        # the cache the wrapper wrote is the oracle's cache (layer 0: embedding, norm, projection, rotary only)
        got_k, want_k = store.key_cache[0].cpu().float(), kc[0].float()
        pair = torch.sqrt(want_k[..., :64] ** 2 + want_k[..., 64:] ** 2).repeat(1, 1, 1, 2)
        rel = ((got_k - want_k).abs() / pair.clamp(min=1e-3))
        print(f"layer 0 key cache vs oracle: worst |d| / pair length {float(rel.max()):.4f}, "
              f"{int((rel > 2.0 ** -7).sum())} of {rel.numel()} beyond 2^-7", flush=True)
        assert bool(((got_k - want_k).abs() <= 2.0 ** -6 * pair + 1e-6).all()), "layer 0 key cache vs oracle"
    finally:
        remove_qwen3_moe_patches()
        if had is None:
            try:
                del ALL_ATTENTION_FUNCTIONS._global_mapping["triton-invariant"]
            except Exception:
                pass
        else:
            ALL_ATTENTION_FUNCTIONS["triton-invariant"] = had


def test_huggingface_decode_step_captured_the_way_the_reference_captures_it():
    """The reference's CudaGraphManager (vexact/inferencer/cudagraph_utils.py:108-176) warms the model up and captures
    it on static buffers with an even split of the bucket's tokens, no cache writes and max_seqlen_q = the bucket's
    tokens; a step then copies its metadata in, padded (inferencer.py:293-349: zeroed ids and positions, slot -1,
    zero-length padded requests whose query_start_loc is the real token count, block tables 0) and replays. The
    same procedure on the HIP kernels: replays of a 4-token / 4-request bucket give the bits of the eager,
    unpadded steps, for three and for two requests, and write the cache the eager step writes."""
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    from vexact_amd.batch_invariant_ops import flash_attention_forward, set_batch_invariant_mode
    from vexact_amd.batch_invariant_ops.kv_cache_context import (KVCacheManager, KVCacheStore, clear_kv_cache_context,
                                                                 set_kv_cache_context)
    from vexact_amd.decoder import build_step_metadata
    from vexact_amd.models.qwen3_moe import apply_qwen3_moe_patches, remove_qwen3_moe_patches

    page, max_blocks_per_req, cap_t, cap_s = 16, 32, 4, 4
    cache_cfg = types.SimpleNamespace(page_size=page, max_cache_blocks=64)
    had = ALL_ATTENTION_FUNCTIONS._global_mapping.get("triton-invariant") if hasattr(ALL_ATTENTION_FUNCTIONS, "_global_mapping") else None
    ALL_ATTENTION_FUNCTIONS["triton-invariant"] = flash_attention_forward
    apply_qwen3_moe_patches()
    try:
        hf_cfg, model = _build_model(seed=23)
        model = model.cuda()
        store = KVCacheStore(hf_cfg, cache_cfg, torch.device("cuda"))
        alloc = KVCacheManager(cache_cfg)
        rng = np.random.default_rng(24)
        lens = [21, 70, 9]
        prompts = [rng.integers(0, hf_cfg.vocab_size, size=n) for n in lens]
        blocks = [list(alloc.allocate_blocks(n + 2, 0)) for n in lens]

        def forward(ids, positions):
            out = model.model(input_ids=ids, position_ids=positions, use_cache=False, return_dict=True)
            return model.lm_head(out.last_hidden_state)

        def eager(which, new_tokens, ids):
            reqs = [dict(num_computed_tokens=done, tokens_this_step=new, block_ids=blocks[s])
                    for s, (done, new) in zip(which, new_tokens)]
            meta = build_step_metadata(reqs, page, max_blocks_per_req)
            dev = {k: torch.as_tensor(v).cuda() for k, v in meta.items() if k != "max_seqlen_q"}
            set_kv_cache_context(is_paged_attn=True, key_cache=store.key_cache, value_cache=store.value_cache,
                                 block_tables=dev["block_tables"], context_lens=dev["context_lens"],
                                 slot_mapping=dev["slot_mapping"], query_start_loc=dev["query_start_loc"],
                                 max_seqlen_q=int(meta["max_seqlen_q"]))
            try:
                with torch.inference_mode(), set_batch_invariant_mode(True):
                    logits = forward(torch.as_tensor(ids)[None].cuda(), dev["positions"][None])
                    last = (dev["query_start_loc"][1:] - 1).long()
                    return logits[0, last, :].clone(), meta
            finally:
                clear_kv_cache_context()

        plogits, _ = eager([0, 1, 2], [(n, n) for n in lens], np.concatenate(prompts))
        first = plogits.argmax(-1).cpu().numpy()

        # ---- static buffers of the bucket and the capture, as CudaGraphManager.capture does it
        i32 = dict(dtype=torch.int32, device="cuda")
        ids_s = torch.zeros(1, cap_t, dtype=torch.int64, device="cuda")
        pos_s = torch.zeros(1, cap_t, dtype=torch.int64, device="cuda")
        bt_s = torch.zeros(cap_s, max_blocks_per_req, **i32)
        ctx_s = torch.zeros(cap_s, **i32)
        slot_s = torch.full((cap_t,), -1, **i32)
        qsl_s = torch.zeros(cap_s + 1, **i32)
        per = torch.full((cap_s,), cap_t // cap_s, **i32)
        per[: cap_t % cap_s] += 1
        qsl_s[1:] = per.cumsum(0)
        ctx_s.copy_(per)
        set_kv_cache_context(is_paged_attn=True, key_cache=store.key_cache, value_cache=store.value_cache, block_tables=bt_s,
                             context_lens=ctx_s, slot_mapping=slot_s, query_start_loc=qsl_s, max_seqlen_q=cap_t)
        kcaches = list(store.key_cache.values()) if isinstance(store.key_cache, dict) else list(store.key_cache)
        cache_before = [t.clone() for t in kcaches]
        graph = torch.cuda.CUDAGraph()
        try:
            with torch.inference_mode(), set_batch_invariant_mode(True):
                forward(ids_s, pos_s)  # warm-up
                with torch.cuda.graph(graph):
                    out_s = forward(ids_s, pos_s)
        finally:
            clear_kv_cache_context()
        for a, b in zip(kcaches, cache_before):
            assert_bitwise(a, b, "capture and warm-up write nothing into the cache (slot -1)")

        def replay(which, ids):
            reqs = [dict(num_computed_tokens=lens[s] + 1, tokens_this_step=1, block_ids=blocks[s]) for s in which]
            meta = build_step_metadata(reqs, page, max_blocks_per_req)
            n = len(which)
            ids_s.zero_(); pos_s.zero_(); bt_s.fill_(-1); ctx_s.zero_(); slot_s.fill_(-1); qsl_s.zero_()
            bt_s[:n].copy_(torch.as_tensor(meta["block_tables"]))
            ctx_s[:n].copy_(torch.as_tensor(meta["context_lens"]))
            slot_s[:n].copy_(torch.as_tensor(meta["slot_mapping"]))
            qsl_s[: n + 1].copy_(torch.as_tensor(meta["query_start_loc"]))
            if cap_s > n:
                bt_s[n:].zero_()
                qsl_s[n + 1:] = n
            ids_s[0, :n].copy_(torch.as_tensor(ids))
            pos_s[0, :n].copy_(torch.as_tensor(meta["positions"]))
            graph.replay()
            torch.cuda.synchronize()
            return out_s[0, :n, :].clone()

        for which in ([0, 1, 2], [2, 0]):
            store_before = [t.clone() for t in kcaches]
            want, _ = eager(which, [(lens[s] + 1, 1) for s in which], first[which])
            k_eager = [t.clone() for t in kcaches]
            for t, b in zip(kcaches, store_before):
                t.copy_(b)
            got = replay(which, first[which])
            assert_bitwise(got, want, f"graph replay of requests {which} in a 4 / 4 bucket vs the eager unpadded step")
            for a, b in zip(kcaches, k_eager):
                assert_bitwise(a, b, "the replay writes the keys the eager step writes")
    finally:
        remove_qwen3_moe_patches()
        if had is None:
            try:
                del ALL_ATTENTION_FUNCTIONS._global_mapping["triton-invariant"]
            except Exception:
                pass
        else:
            ALL_ATTENTION_FUNCTIONS["triton-invariant"] = had


def test_fused_rms_norm_patch_gives_the_bits_of_the_unfused_forward():
    # Qwen3MoeRMSNorm.forward replaced by one kernel: hidden-size rows and head-size rows (q / k norm), bf16 and fp16,
    # against HuggingFace's own forward run under batch-invariant mode
    from transformers.models.qwen3_moe import modeling_qwen3_moe as hf

    from vexact_amd.batch_invariant_ops import set_batch_invariant_mode
    from vexact_amd.models.qwen3_moe import apply_qwen3_moe_patches, remove_qwen3_moe_patches
    from vexact_amd.models.qwen3_moe.modeling_qwen3_moe import fused_rms_norm_forward

    original = hf.Qwen3MoeRMSNorm.forward
    apply_qwen3_moe_patches()
    try:
        assert hf.Qwen3MoeRMSNorm.forward is fused_rms_norm_forward
        g = torch.Generator().manual_seed(3)
        for shape, dtype in (((1, 37, 2048), BF), ((1, 9, 32, 128), BF), ((256, 2048), BF), ((1, 5, 4, 128), torch.float16),
                             ((3, 200), BF)):
            norm = hf.Qwen3MoeRMSNorm(shape[-1], eps=1e-6)
            with torch.no_grad():
                norm.weight.copy_(1.0 + 0.2 * torch.randn(shape[-1], generator=g))
            norm = norm.to(dtype).cuda()
            x = (3.0 * torch.randn(shape, generator=g)).to(dtype).cuda()
            with torch.inference_mode(), set_batch_invariant_mode(True):
                fused = norm(x)
                unfused = original(norm, x)
            assert fused.shape == unfused.shape and fused.dtype == unfused.dtype
            assert_bitwise(fused, unfused, f"fused RMSNorm forward, shape {shape}, {dtype}")
            with torch.inference_mode():  # outside the mode the original forward runs
                assert_bitwise(norm(x), original(norm, x), "outside batch-invariant mode")
        # Rows of small and of large entries sweep the argument of the reciprocal square root over many binades: the
        # kernel's HuggingFace form uses the device library's rsqrt, the operation torch.rsqrt runs on this device,
        # so every element has the unfused forward's bits (1 / sqrt differs from it by an fp32 ulp now and then, which
        # used to move about one output element in 10^5 to the neighbouring bf16 value)
        for n in (64, 320, 2048):
            norm = hf.Qwen3MoeRMSNorm(n, eps=1e-6).to(BF).cuda()
            for scale in (0.05, 1.0, 30.0, 1e-3):
                x = (scale * torch.randn(600, n, generator=g)).to(BF).cuda()
                with torch.inference_mode(), set_batch_invariant_mode(True):
                    fused, unfused = norm(x), original(norm, x)
                assert_bitwise(fused, unfused, f"fused RMSNorm forward on rows of scale {scale}, n={n}")
        # with autograd the same kernel runs (the trainer's forward is the rollout's), and its backward is the
        # derivative of the original forward
        norm = hf.Qwen3MoeRMSNorm(256, eps=1e-6)
        with torch.no_grad():
            norm.weight.copy_(1.0 + 0.2 * torch.randn(256, generator=g))
        norm = norm.to(BF).cuda()
        x = torch.randn(2, 50, 256, generator=g).to(BF).cuda()
        dy = torch.randn(2, 50, 256, generator=g).to(BF).cuda()
        with torch.inference_mode(), set_batch_invariant_mode(True):
            rollout = norm(x)
        xa = x.clone().requires_grad_()
        with set_batch_invariant_mode(True):
            ya = norm(xa)
        assert_bitwise(ya.detach(), rollout, "forward under autograd")
        ya.backward(dy)
        got_x, got_w = xa.grad, norm.weight.grad.clone()
        norm.weight.grad = None
        xb = x.clone().requires_grad_()
        original(norm, xb).backward(dy)
        for name, a, b in (("input", got_x, xb.grad), ("weight", got_w, norm.weight.grad)):
            err, scale = (a.float() - b.float()).abs(), float(b.float().abs().max())
            assert float(err.max()) <= 2e-2 * scale, f"RMSNorm gradient of the {name}: {float(err.max()):.4g} vs scale {scale:.4g}"
    finally:
        remove_qwen3_moe_patches()
    assert hf.Qwen3MoeRMSNorm.forward is original


def test_fused_rope_patch_gives_the_bits_of_apply_rotary_pos_emb():
    from transformers.models.qwen3_moe import modeling_qwen3_moe as hf

    from vexact_amd.models.qwen3_moe import apply_qwen3_moe_patches, remove_qwen3_moe_patches
    from vexact_amd.models.qwen3_moe.modeling_qwen3_moe import fused_apply_rotary_pos_emb

    original = hf.apply_rotary_pos_emb
    apply_qwen3_moe_patches()
    try:
        assert hf.apply_rotary_pos_emb is fused_apply_rotary_pos_emb
        g = torch.Generator().manual_seed(5)
        for B, T, Hq, Hkv, D in ((1, 300, 32, 4, 128), (1, 1, 4, 2, 128), (3, 17, 8, 8, 64), (1, 40, 6, 2, 96)):
            # the attention module's layout: projections [B, T, heads, D] seen as [B, heads, T, D]
            q = (2.0 * torch.randn(B, T, Hq, D, generator=g)).to(BF).cuda().transpose(1, 2)
            k = (2.0 * torch.randn(B, T, Hkv, D, generator=g)).to(BF).cuda().transpose(1, 2)
            ang = 50.0 * torch.rand(B, T, D // 2, generator=g)
            cos = torch.cat([ang.cos(), ang.cos()], -1).to(BF).cuda()
            sin = torch.cat([ang.sin(), ang.sin()], -1).to(BF).cuda()
            with torch.inference_mode():
                fq, fk = hf.apply_rotary_pos_emb(q, k, cos, sin)
                oq, ok = original(q, k, cos, sin)
            assert fq.shape == oq.shape and fk.shape == ok.shape
            assert_bitwise(fq, oq, f"rotated queries, B={B} T={T} D={D}")
            assert_bitwise(fk, ok, f"rotated keys, B={B} T={T} D={D}")
        # with autograd the kernel runs in both directions: the original's output and gradient bits
        q0 = (2.0 * torch.randn(1, 50, 8, 128, generator=g)).to(BF).cuda()
        k0 = (2.0 * torch.randn(1, 50, 2, 128, generator=g)).to(BF).cuda()
        ang = 50.0 * torch.rand(1, 50, 64, generator=g)
        cos, sin = torch.cat([ang.cos(), ang.cos()], -1).to(BF).cuda(), torch.cat([ang.sin(), ang.sin()], -1).to(BF).cuda()
        dq, dk = torch.randn(1, 8, 50, 128, generator=g).to(BF).cuda(), torch.randn(1, 2, 50, 128, generator=g).to(BF).cuda()
        grads = []
        for fn in (hf.apply_rotary_pos_emb, original):
            ql, kl = q0.clone().requires_grad_(), k0.clone().requires_grad_()
            oq, ok = fn(ql.transpose(1, 2), kl.transpose(1, 2), cos, sin)
            torch.autograd.backward([oq, ok], [dq, dk])
            grads.append((oq.detach(), ok.detach(), ql.grad, kl.grad))
        for name, a, b in zip(("rotated queries", "rotated keys", "query gradient", "key gradient"), *grads):
            assert_bitwise(a, b, f"{name} under autograd")
        # what the kernel does not take falls through to the original (fp32 here)
        q = torch.randn(1, 2, 5, 64, device="cuda"); k = torch.randn(1, 2, 5, 64, device="cuda")
        cos = torch.randn(1, 5, 64, device="cuda"); sin = torch.randn(1, 5, 64, device="cuda")
        fq, fk = hf.apply_rotary_pos_emb(q, k, cos, sin)
        oq, ok = original(q, k, cos, sin)
        assert torch.equal(fq, oq) and torch.equal(fk, ok)
    finally:
        remove_qwen3_moe_patches()
    assert hf.apply_rotary_pos_emb is original



def test_fused_attention_and_residual_patches_give_the_bits_of_the_unfused_forwards():
    # Qwen3MoeAttention.forward over the paged cache as one q/k/v projection + one norm/rotary/store kernel + attention,
    # and Qwen3MoeDecoderLayer.forward with its residual additions inside the norm and the MoE combine, against
    # HuggingFace's own forwards (three projections, q / k norm, apply_rotary_pos_emb, the registered attention
    # function's cache write, two additions): logits and both layers' caches, for a packed prefill of three prompts
    # and a decode step
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS
    from transformers.models.qwen3_moe import modeling_qwen3_moe as hf

    from vexact_amd.batch_invariant_ops import flash_attention_forward, set_batch_invariant_mode
    from vexact_amd.batch_invariant_ops.kv_cache_context import KVCacheStore, clear_kv_cache_context, set_kv_cache_context
    from vexact_amd.decoder import build_step_metadata
    from vexact_amd.models.qwen3_moe import apply_qwen3_moe_patches, fuse_qkv_weights, remove_qwen3_moe_patches, unfuse_qkv_weights
    from vexact_amd.models.qwen3_moe.modeling_qwen3_moe import fused_attention_forward, fused_decoder_layer_forward

    page, max_blocks_per_req = 16, 16
    cache_cfg = types.SimpleNamespace(page_size=page, max_cache_blocks=40)
    had = ALL_ATTENTION_FUNCTIONS._global_mapping.get("triton-invariant") if hasattr(ALL_ATTENTION_FUNCTIONS, "_global_mapping") else None
    ALL_ATTENTION_FUNCTIONS["triton-invariant"] = flash_attention_forward
    original, original_layer = hf.Qwen3MoeAttention.forward, hf.Qwen3MoeDecoderLayer.forward
    apply_qwen3_moe_patches()
    try:
        assert hf.Qwen3MoeAttention.forward is fused_attention_forward
        assert hf.Qwen3MoeDecoderLayer.forward is fused_decoder_layer_forward
        hf_cfg, model = _build_model(seed=23)
        model = model.cuda()
        rng = np.random.default_rng(24)
        lens = [37, 5, 120]
        prompts = [rng.integers(0, hf_cfg.vocab_size, size=n) for n in lens]
        blocks, nxt = [], 0
        for n in lens:
            need = -(-(n + 1) // page)
            blocks.append(list(range(nxt, nxt + need)))
            nxt += need

        def run(fused, which_store):
            hf.Qwen3MoeAttention.forward = fused_attention_forward if fused else original
            hf.Qwen3MoeDecoderLayer.forward = fused_decoder_layer_forward if fused else original_layer
            outs = []
            for new_tokens, ids in (([(n, n) for n in lens], np.concatenate(prompts)), ([(n + 1, 1) for n in lens], np.array([3, 1, 4]))):
                reqs = [dict(num_computed_tokens=done, tokens_this_step=new, block_ids=blocks[s]) for s, (done, new) in enumerate(new_tokens)]
                meta = build_step_metadata(reqs, page, max_blocks_per_req)
                dev = {k: torch.as_tensor(v).cuda() for k, v in meta.items() if k != "max_seqlen_q"}
                set_kv_cache_context(is_paged_attn=True, key_cache=which_store.key_cache, value_cache=which_store.value_cache,
                                     block_tables=dev["block_tables"], context_lens=dev["context_lens"],
                                     slot_mapping=dev["slot_mapping"], query_start_loc=dev["query_start_loc"],
                                     max_seqlen_q=int(meta["max_seqlen_q"]))
                try:
                    with torch.inference_mode(), set_batch_invariant_mode(True):
                        out = model.model(input_ids=torch.as_tensor(ids)[None].cuda(), position_ids=dev["positions"][None],
                                          use_cache=False, return_dict=True)
                        outs.append(model.lm_head(out.last_hidden_state)[0].clone())
                finally:
                    clear_kv_cache_context()
            return outs

        stores = [KVCacheStore(hf_cfg, cache_cfg, torch.device("cuda")) for _ in range(2)]
        for s in stores:
            for t in list(s.key_cache.values()) + list(s.value_cache.values()):
                t.zero_()
        unfused = run(False, stores[0])
        attn = model.model.layers[0].self_attn
        ptrs = [p_.data_ptr() for p_ in (attn.q_proj.weight, attn.k_proj.weight, attn.v_proj.weight)]
        fused = run(True, stores[1])   # three projections into one buffer: a forward never touches the parameters
        assert [p_.data_ptr() for p_ in (attn.q_proj.weight, attn.k_proj.weight, attn.v_proj.weight)] == ptrs
        assert getattr(attn, "_vx_qkv_weight", None) is None

        def same_as_unfused(got, what):
            for name, a, b in zip(("prefill", "decode"), got, unfused):
                assert_bitwise(a, b, f"{name} logits, fused attention forward ({what}) vs HuggingFace's")
            for layer in range(2):
                assert_bitwise(stores[1].key_cache[layer], stores[0].key_cache[layer], f"key cache of layer {layer} ({what})")
                assert_bitwise(stores[1].value_cache[layer], stores[0].value_cache[layer], f"value cache of layer {layer} ({what})")

        same_as_unfused(fused, "separate weights")
        # the explicit load-time step: one weight tensor per module, the parameters its row ranges
        before = {k: v.clone() for k, v in model.state_dict().items()}
        assert fuse_qkv_weights(model) == len(model.model.layers)
        assert attn.q_proj.weight.data_ptr() == attn._vx_qkv_weight.data_ptr(), "the parameters are views of the fused weight"
        after = model.state_dict()
        assert list(after) == list(before) and all(torch.equal(after[k], before[k]) for k in before), "state_dict values"
        same_as_unfused(run(True, stores[1]), "one weight")
        # a parameter written in place (what a weight synchronisation does) reaches the fused weight; one that gets
        # new storage takes the module back to three projections
        with torch.no_grad():
            attn.v_proj.weight.data.mul_(0.5)
        again_fused, again_unfused = run(True, stores[1]), run(False, stores[0])
        assert_bitwise(again_fused[1], again_unfused[1], "after an in-place weight update")
        assert not torch.equal(again_fused[1], fused[1])
        model.load_state_dict(before)   # in place as well: copies into the fused storage
        assert attn.q_proj.weight.data_ptr() == attn._vx_qkv_weight.data_ptr()
        unfused = run(False, stores[0])
        same_as_unfused(run(True, stores[1]), "after load_state_dict")
        attn.v_proj.weight.data = attn.v_proj.weight.data.clone() * 2
        again_fused, again_unfused = run(True, stores[1]), run(False, stores[0])
        assert_bitwise(again_fused[1], again_unfused[1], "after a parameter got new storage")
        # and back: storages of their own again, which is what safetensors' save_file insists on
        assert unfuse_qkv_weights(model) == len(model.model.layers)
        qkv = (attn.q_proj.weight, attn.k_proj.weight, attn.v_proj.weight)
        assert len({w.untyped_storage().data_ptr() for w in qkv}) == 3 and attn._vx_qkv_weight is None
        from safetensors.torch import save
        assert len(save({k: v for k, v in model.state_dict().items() if "self_attn" in k})) > 0
        assert_bitwise(run(True, stores[1])[1], again_unfused[1], "after unfusing")
    finally:
        hf.Qwen3MoeAttention.forward = fused_attention_forward  # what remove_qwen3_moe_patches expects to undo
        hf.Qwen3MoeDecoderLayer.forward = fused_decoder_layer_forward
        remove_qwen3_moe_patches()
        if had is None:
            try:
                del ALL_ATTENTION_FUNCTIONS._global_mapping["triton-invariant"]
            except Exception:
                pass
        else:
            ALL_ATTENTION_FUNCTIONS["triton-invariant"] = had
    assert hf.Qwen3MoeAttention.forward is original and hf.Qwen3MoeDecoderLayer.forward is original_layer


def _fp32_reference_logits(P, ids, lens, selected, cfg):
    """The tiny model in plain fp32 tensor operations on the CPU (autograd-friendly): RMSNorm, q/k/v, per-head norm,
    rotary embedding, causal attention per sequence with grouped kv heads, the MoE block on the GPU's expert choice."""
    Hq, Hkv, D, k = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.num_experts_per_tok

    def rms(x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + cfg.rms_norm_eps) * w

    def rot(x, cos, sin):
        x1, x2 = x[..., : D // 2], x[..., D // 2:]
        return x * cos[:, None, :] + torch.cat([-x2, x1], -1) * sin[:, None, :]

    T = len(ids)
    h = P["model.embed_tokens.weight"][torch.as_tensor(ids)]
    pos = torch.cat([torch.arange(n) for n in lens]).float()
    inv = 1.0 / (1.0e6 ** (torch.arange(0, D, 2).float() / D))
    ang = pos[:, None] * inv[None, :]
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1), torch.cat([ang.sin(), ang.sin()], -1)
    for l in range(cfg.num_hidden_layers):
        pre = f"model.layers.{l}."
        x = rms(h, P[pre + "input_layernorm.weight"])
        q = (x @ P[pre + "self_attn.q_proj.weight"].t()).view(T, Hq, D)
        kk = (x @ P[pre + "self_attn.k_proj.weight"].t()).view(T, Hkv, D)
        v = (x @ P[pre + "self_attn.v_proj.weight"].t()).view(T, Hkv, D)
        q, kk = rot(rms(q, P[pre + "self_attn.q_norm.weight"]), cos, sin), rot(rms(kk, P[pre + "self_attn.k_norm.weight"]), cos, sin)
        outs, o = [], 0
        for n in lens:
            qs = q[o:o + n].transpose(0, 1)                                        # [Hq, n, D]
            ks = kk[o:o + n].transpose(0, 1).repeat_interleave(Hq // Hkv, dim=0)
            vs = v[o:o + n].transpose(0, 1).repeat_interleave(Hq // Hkv, dim=0)
            s = (qs @ ks.transpose(1, 2)) * D ** -0.5
            s = s.masked_fill(torch.ones(n, n, dtype=torch.bool).triu(1), float("-inf"))
            outs.append((torch.softmax(s, -1) @ vs).transpose(0, 1).reshape(n, Hq * D))
            o += n
        h = h + torch.cat(outs) @ P[pre + "self_attn.o_proj.weight"].t()
        x = rms(h, P[pre + "post_attention_layernorm.weight"])
        probs = torch.softmax(x @ P[pre + "mlp.gate.weight"].t(), -1)
        sel = selected[l]
        w = probs.gather(-1, sel)
        w = w / w.sum(-1, keepdim=True)
        gu, dn = P[pre + "mlp.experts.gate_up_proj"], P[pre + "mlp.experts.down_proj"]
        inter = gu.shape[1] // 2
        moe = torch.zeros_like(h)
        for i in range(k):
            e = sel[:, i]
            gate = torch.einsum("th,tih->ti", x, gu[e, :inter])
            up = torch.einsum("th,tih->ti", x, gu[e, inter:])
            moe = moe + w[:, i: i + 1] * torch.einsum("ti,thi->th", torch.nn.functional.silu(gate) * up, dn[e])
        h = h + moe
    return rms(h, P["model.norm.weight"]) @ P["lm_head.weight"].t()


def test_training_forward_gives_the_rollout_bits_and_its_gradients_match_an_fp32_model():
    """The property the reference exists for: the trainer's forward (packed sequences, no cache, autograd on, the packed
    attention and fused-MoE autograd functions) reproduces the rollout's logits (paged prefill, inference mode, every fused
    patch) bit for bit, so on-policy logprobs are exact; and its backward gives the gradients of the model (against the
    same model in fp32 tensor operations on the CPU, following the GPU's expert choice), router weights included."""
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    from vexact_amd.batch_invariant_ops import flash_attention_forward, set_batch_invariant_mode
    from vexact_amd.batch_invariant_ops.kv_cache_context import KVCacheStore, clear_kv_cache_context, set_kv_cache_context
    from vexact_amd.batch_invariant_ops.standalone_logprobs import logprobs_from_logits_flash_attn
    from vexact_amd.decoder import build_step_metadata
    from vexact_amd.models.qwen3_moe import apply_qwen3_moe_patches, remove_qwen3_moe_patches

    page = 16
    cache_cfg = types.SimpleNamespace(page_size=page, max_cache_blocks=40)
    had = ALL_ATTENTION_FUNCTIONS._global_mapping.get("triton-invariant") if hasattr(ALL_ATTENTION_FUNCTIONS, "_global_mapping") else None
    ALL_ATTENTION_FUNCTIONS["triton-invariant"] = flash_attention_forward
    apply_qwen3_moe_patches()
    try:
        hf_cfg, model = _build_model(seed=31)
        model = model.cuda()
        rng = np.random.default_rng(32)
        lens = [37, 5, 120]
        ids = np.concatenate([rng.integers(0, hf_cfg.vocab_size, size=n) for n in lens])
        targets = torch.as_tensor(rng.integers(0, hf_cfg.vocab_size, size=len(ids)))
        ids_d = torch.as_tensor(ids)[None].cuda()
        # ---- rollout: paged prefill in inference mode
        blocks, nxt = [], 0
        for n in lens:
            blocks.append(list(range(nxt, nxt + -(-n // page))))
            nxt += len(blocks[-1])
        meta = build_step_metadata([dict(num_computed_tokens=n, tokens_this_step=n, block_ids=b) for n, b in zip(lens, blocks)], page, 16)
        dev = {k: torch.as_tensor(v).cuda() for k, v in meta.items() if k != "max_seqlen_q"}
        store = KVCacheStore(hf_cfg, cache_cfg, torch.device("cuda"))
        set_kv_cache_context(is_paged_attn=True, key_cache=store.key_cache, value_cache=store.value_cache,
                             block_tables=dev["block_tables"], context_lens=dev["context_lens"], slot_mapping=dev["slot_mapping"],
                             query_start_loc=dev["query_start_loc"], max_seqlen_q=int(meta["max_seqlen_q"]))
        try:
            with torch.inference_mode(), set_batch_invariant_mode(True):
                out = model.model(input_ids=ids_d, position_ids=dev["positions"][None], use_cache=False, return_dict=True)
                rollout = model.lm_head(out.last_hidden_state)[0].clone()
                rollout_lp = logprobs_from_logits_flash_attn(rollout.float(), targets.cuda())
        finally:
            clear_kv_cache_context()
        # ---- trainer: the same tokens as a packed batch, gradients on
        selected = []
        hooks = [l.mlp.experts.register_forward_pre_hook(lambda mod, args, kw: selected.append(kw["selected_experts"].detach().cpu()),
                                                         with_kwargs=True) for l in model.model.layers]
        for p in model.parameters():
            p.requires_grad_(True)
        set_kv_cache_context(is_paged_attn=False, context_lens=dev["context_lens"], query_start_loc=dev["query_start_loc"],
                             max_seqlen_q=int(meta["max_seqlen_q"]))
        try:
            with set_batch_invariant_mode(True):
                out = model.model(input_ids=ids_d, position_ids=dev["positions"][None], use_cache=False, return_dict=True)
                logits = model.lm_head(out.last_hidden_state)[0]
                assert logits.requires_grad
                assert_bitwise(logits.detach(), rollout, "trainer's logits vs the rollout's")
                lp = logprobs_from_logits_flash_attn(logits.float(), targets.cuda(), inplace_backward=True)
                assert_bitwise(lp.detach(), rollout_lp, "trainer's logprobs vs the rollout's")
                (-lp.sum()).backward()
        finally:
            clear_kv_cache_context()
            for h in hooks:
                h.remove()
        # ---- the same model in fp32 on the CPU
        P = {n: p.detach().cpu().float().requires_grad_() for n, p in model.named_parameters()}
        ref_logits = _fp32_reference_logits(P, ids, lens, selected, hf_cfg)
        ref_lp = torch.log_softmax(ref_logits, -1).gather(-1, targets[:, None])[:, 0]
        assert float((lp.detach().cpu() - ref_lp.detach()).abs().max()) <= 0.1, "logprobs vs the fp32 model"
        (-ref_lp.sum()).backward()
        worst = []
        for n, p in model.named_parameters():
            assert p.grad is not None, f"no gradient for {n}"
            want = P[n].grad
            err, scale = (p.grad.detach().cpu().float() - want).abs(), float(want.abs().max())
            worst.append((float(err.max()) / max(scale, 1e-12), n))
            assert float(err.max()) <= 0.08 * scale + 1e-6 and float(err.mean()) <= 0.01 * scale + 1e-7, (
                f"grad of {n}: max err {float(err.max()):.4g}, mean {float(err.mean()):.4g}, scale {scale:.4g}")
        worst.sort(reverse=True)
        print("largest gradient errors relative to the largest entry:", [(round(e, 4), n) for e, n in worst[:4]], flush=True)
    finally:
        remove_qwen3_moe_patches()
        if had is None:
            try:
                del ALL_ATTENTION_FUNCTIONS._global_mapping["triton-invariant"]
            except Exception:
                pass
        else:
            ALL_ATTENTION_FUNCTIONS["triton-invariant"] = had
