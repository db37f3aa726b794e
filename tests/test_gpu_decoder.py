"""GPU parity of the whole decoder step: a tiny Qwen3-MoE-shaped model against the CPU oracle,
batch-1 vs batch-N logprob bits, prefill vs decode bits, and HIP-graph replay (padded bucket)
vs eager (the assertions of tests/test_inferencer.py:300-595, atol = 0)."""

import numpy as np
import pytest
import torch

from oracle import decoder as OD
from tests.util import assert_bf16_close, assert_bitwise, bf16_ulp_distance

pytestmark = pytest.mark.gpu

from vexact_amd.decoder import (  # noqa: E402
    DecoderWeights,
    Qwen3MoeDecoder,
    build_step_metadata,
    tiny_config,
)


def _setup(num_seqs=5, seed=3, layers=2):
    cfg = tiny_config(num_layers=layers)
    w = DecoderWeights(cfg, device="cuda", seed=seed, std=0.05, norm_std=0.1)  # every norm weight differs from 1
    rng = np.random.default_rng(seed)
    prompt_lens = rng.integers(5, 300, size=num_seqs)
    prompts = [rng.integers(0, cfg.vocab_size, size=n) for n in prompt_lens]
    pages = [(n + 2 + cfg.page_size - 1) // cfg.page_size for n in prompt_lens]
    perm = rng.permutation(sum(pages) + 7)
    blocks, o = [], 0
    for p in pages:
        blocks.append(perm[o : o + p].tolist())
        o += p
    dec = Qwen3MoeDecoder(cfg, w, num_cache_blocks=len(perm))
    return cfg, w, dec, prompts, blocks


def _prefill(dec, cfg, prompts, blocks, which, routing_log=None):
    reqs = [dict(num_computed_tokens=len(prompts[s]), tokens_this_step=len(prompts[s]), block_ids=blocks[s]) for s in which]
    meta = build_step_metadata(reqs, cfg.page_size, (cfg.max_model_len + cfg.page_size - 1) // cfg.page_size)
    ids = np.concatenate([prompts[s] for s in which])
    b = dec.bucket(len(ids), len(which))
    b.load(meta, ids)
    dec.step(b, meta["max_seqlen_q"], routing_log)
    torch.cuda.synchronize()
    return b.tokens.cpu().clone(), b.logprobs.cpu().clone(), meta, ids


def _decode_meta(cfg, prompts, blocks, which):
    reqs = [dict(num_computed_tokens=len(prompts[s]) + 1, tokens_this_step=1, block_ids=blocks[s]) for s in which]
    return build_step_metadata(reqs, cfg.page_size, (cfg.max_model_len + cfg.page_size - 1) // cfg.page_size)


def _check_routing_report(report, what):
    # the oracle may only be forced across near-ties: a few bf16 ulps of the router logits
    tot = sum(r["tokens"] for r in report)
    dif = sum(r["differ"] for r in report)
    print(f"{what}: routing differed on {dif} of {tot} (token, layer) pairs; "
          f"largest logit gap crossed {max(r['max_gap'] for r in report):.4f}")
    assert dif <= 0.1 * tot, f"{what}: routing differs on too many tokens"
    assert max(r["max_gap_rel"] for r in report) <= 0.05 or max(r["max_gap"] for r in report) <= 0.05, (
        f"{what}: forced routing crossed a logit gap that is not a near-tie")


def test_tiny_decoder_matches_cpu_oracle_and_is_batch_invariant():
    cfg, w, dec, prompts, blocks = _setup()
    allseq = list(range(len(prompts)))
    rlog = []
    tok, lp, meta, ids = _prefill(dec, cfg, prompts, blocks, allseq, rlog)

    # CPU oracle on the same input bits, following the GPU's expert choice at near-ties
    wc = w.to_cpu()
    cos, sin = OD.rope_tables_ref(cfg.head_dim, cfg.rope_theta, cfg.max_model_len)  # the oracle's own tables
    kc = [torch.zeros(t.shape, dtype=t.dtype) for t in dec.key_cache]
    vc = [torch.zeros(t.shape, dtype=t.dtype) for t in dec.value_cache]
    report = []
    logits_ref, _, _ = OD.decoder_step_ref(cfg, wc, ids, meta, kc, vc, cos, sin, [r.cpu() for r in rlog], report)
    _check_routing_report(report, "prefill")
    lp_at_gpu_tok = torch.log_softmax(logits_ref.float(), -1).gather(-1, tok.view(-1, 1)).squeeze(-1)
    assert (lp - lp_at_gpu_tok).abs().max() <= 2e-2, "prefill logprob vs CPU oracle"
    # written caches: layer 0 depends on embedding, norm, projection and rotary only
    # a rotated key element is k_j cos -+ k_(j+D/2) sin: where the two products cancel, a one-ulp difference of
    # the projection (fp32 summation order) is many ulps of the small result, so the bound for an element is
    # 2 of its own ulps or 2 ulps (2^-7) of its rotation pair's length, which the rotation preserves
    got_k, want_k = dec.key_cache[0].cpu().float(), kc[0].float()
    half = cfg.head_dim // 2
    pair = torch.sqrt(want_k[..., :half] ** 2 + want_k[..., half:] ** 2).repeat(1, 1, 1, 2)
    ok = (bf16_ulp_distance(dec.key_cache[0], kc[0]) <= 2) | ((got_k - want_k).abs() <= 2.0 ** -7 * pair)
    assert bool(ok.all()), f"layer 0 key cache: {int((~ok).sum())} elements beyond 2 ulp of their rotation pair"
    assert_bf16_close(dec.value_cache[0], vc[0], max_ulp=2, what="layer 0 value cache")
    for li in range(1, cfg.num_layers):
        d = (dec.key_cache[li].cpu().float() - kc[li].float()).abs().max()
        assert d <= 0.06 * max(1.0, float(kc[li].float().abs().max())), f"layer {li} key cache"

    # decode step: batch of 5 vs each request alone, eager; 0 differing bits
    first = tok.numpy()
    dmeta = _decode_meta(cfg, prompts, blocks, allseq)
    b = dec.bucket(len(allseq), len(allseq))
    b.load(dmeta, first)
    rlog = []
    dec.step(b, 1, rlog)
    torch.cuda.synchronize()
    lp_batch, tok_batch = b.logprobs.cpu().clone(), b.tokens.cpu().clone()
    for s in allseq:
        m1 = _decode_meta(cfg, prompts, blocks, [s])
        b1 = dec.bucket(1, 1)
        b1.load(m1, first[s : s + 1])
        dec.step(b1, 1)
        torch.cuda.synchronize()
        assert_bitwise(b1.logprobs.cpu(), lp_batch[s : s + 1], f"decode logprob of request {s}: batch 1 vs batch 5")
        assert int(b1.tokens[0]) == int(tok_batch[s])

    # oracle decode step
    report = []
    logits_ref, _, _ = OD.decoder_step_ref(cfg, wc, first, dmeta, kc, vc, cos, sin, [r.cpu() for r in rlog], report)
    _check_routing_report(report, "decode")
    lp_ref = torch.log_softmax(logits_ref.float(), -1).gather(-1, tok_batch.view(-1, 1)).squeeze(-1)
    assert (lp_batch - lp_ref).abs().max() <= 2e-2, "decode logprob vs CPU oracle"


def test_prefill_alone_equals_prefill_in_batch_and_chunked():
    cfg, w, dec, prompts, blocks = _setup(seed=4)
    allseq = list(range(len(prompts)))
    tok, lp, _, _ = _prefill(dec, cfg, prompts, blocks, allseq)
    for s in (0, 3):
        t1, l1, _, _ = _prefill(dec, cfg, prompts, blocks, [s])
        assert_bitwise(l1, lp[s : s + 1], f"prefill logprob of request {s}: alone vs batch")
        assert int(t1[0]) == int(tok[s])
    # chunked prefill of request 1: first part, then the rest; last-token logprob must not change
    s = 1
    n = len(prompts[s])
    cut = max(1, n // 2)
    maxb = (cfg.max_model_len + cfg.page_size - 1) // cfg.page_size
    for lo, hi in ((0, cut), (cut, n)):
        meta = build_step_metadata([dict(num_computed_tokens=hi, tokens_this_step=hi - lo, block_ids=blocks[s])], cfg.page_size, maxb)
        b = dec.bucket(hi - lo, 1)
        b.load(meta, prompts[s][lo:hi])
        dec.step(b, meta["max_seqlen_q"])
        torch.cuda.synchronize()
    assert_bitwise(b.logprobs.cpu(), lp[s : s + 1], "chunked prefill vs whole prefill")


def test_graph_replay_with_padding_equals_eager():
    cfg, w, dec, prompts, blocks = _setup(num_seqs=5, seed=5)
    allseq = list(range(5))
    tok, _, _, _ = _prefill(dec, cfg, prompts, blocks, allseq)
    first = tok.numpy()
    dmeta = _decode_meta(cfg, prompts, blocks, allseq)
    be = dec.bucket(5, 5)
    be.load(dmeta, first)
    dec.step(be, 1)
    torch.cuda.synchronize()
    lp_eager, tok_eager = be.logprobs.cpu().clone(), be.tokens.cpu().clone()
    # bucket of 8 tokens / 8 sequences: 3 padded rows
    bg = dec.bucket(8, 8)
    bg.load(dmeta, first)
    g = dec.capture(bg, 1)
    for rep in range(3):
        bg.load(dmeta, first)
        g.replay()
        torch.cuda.synchronize()
        assert_bitwise(bg.logprobs.cpu()[:5], lp_eager, f"graph replay {rep} vs eager")
        assert torch.equal(bg.tokens.cpu()[:5], tok_eager)
        # eager work between replays
        be.load(dmeta, first)
        dec.step(be, 1)
        torch.cuda.synchronize()
        assert_bitwise(be.logprobs.cpu(), lp_eager, "eager repeat")
    # a different, smaller batch through the same graph
    sub = [4, 1]
    m2 = _decode_meta(cfg, prompts, blocks, sub)
    bg.load(m2, first[sub])
    g.replay()
    torch.cuda.synchronize()
    assert_bitwise(bg.logprobs.cpu()[:2], lp_eager[sub], "graph replay with another batch composition")


def test_sampled_decode_is_batch_invariant_and_graph_safe():
    cfg, w, dec, prompts, blocks = _setup(num_seqs=5, seed=7)
    allseq = list(range(5))
    tok, _, _, _ = _prefill(dec, cfg, prompts, blocks, allseq)
    first = tok.numpy()
    sampling = (0.8, 20, 0.9)
    seeds = torch.tensor([11, 22, 33, 44, 55], dtype=torch.int64)
    dmeta = _decode_meta(cfg, prompts, blocks, allseq)
    be = dec.bucket(5, 5)
    be.load(dmeta, first)
    be.seeds.copy_(seeds)
    dec.step(be, 1, sampling=sampling)
    torch.cuda.synchronize()
    tok_e, lp_e = be.tokens.cpu().clone(), be.logprobs.cpu().clone()
    # the token is one of the 20 most likely (bf16 logits tie: everything equal to the 20th value is kept, as in
    # the reference's `logits < kth value` mask) and the logprob is that token's
    logits = be.logits.float().cpu()
    kth = logits.topk(20, dim=-1).values[:, -1]
    assert bool((logits.gather(1, tok_e[:, None].long())[:, 0] >= kth).all())
    want_lp = torch.log_softmax(logits, -1).gather(1, tok_e[:, None])[:, 0]
    assert float((lp_e - want_lp).abs().max()) < 1e-4
    # each request alone draws the same token with the same logprob bits
    b1 = dec.bucket(1, 1)
    for s in allseq:
        b1.load(_decode_meta(cfg, prompts, blocks, [s]), first[s : s + 1])
        b1.seeds.copy_(seeds[s : s + 1])
        dec.step(b1, 1, sampling=sampling)
        torch.cuda.synchronize()
        assert int(b1.tokens[0]) == int(tok_e[s])
        assert_bitwise(b1.logprobs.cpu(), lp_e[s : s + 1], f"sampled logprob of request {s} alone")
    # padded graph replay, twice, and with the requests in another order
    bg = dec.bucket(8, 8)
    bg.load(dmeta, first)
    bg.seeds[:5].copy_(seeds)
    g = dec.capture(bg, 1, sampling=sampling)
    for rep in range(2):
        bg.load(dmeta, first)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(bg.tokens.cpu()[:5], tok_e)
        assert_bitwise(bg.logprobs.cpu()[:5], lp_e, f"sampled graph replay {rep}")
    order = [3, 0, 4, 2, 1]
    bg.load(_decode_meta(cfg, prompts, blocks, order), first[order])
    bg.seeds[:5].copy_(seeds[order])
    g.replay()
    torch.cuda.synchronize()
    assert torch.equal(bg.tokens.cpu()[:5], tok_e[order])


def test_model_with_fragment_order_expert_weights_only_keeps_every_bit(monkeypatch):
    # one copy of the expert weights: prefill (256-row expert tiles on the packed weights instead of 128-row tiles
    # on [E, N, K]) and decode give the bits of the model that keeps both. The model with [E, N, K] tensors is held
    # to 128-row tiles here (the tile height is chosen from the rows per expert, which at 8 experts / top-2 would
    # also give it 256-row tiles), so that the two prefills really run different kernels.
    from vexact_amd import ops
    real = ops.moe_tile_rows
    monkeypatch.setattr(ops, "moe_tile_rows",
                        lambda n, **kw: 128 if not kw.get("packed_only") and real(n, **kw) == 256 else real(n, **kw))
    cfg, w, dec, prompts, blocks = _setup(num_seqs=10, seed=13)
    allseq = list(range(10))
    assert sum(len(p) for p in prompts) > 1024
    tok, lp, meta, ids = _prefill(dec, cfg, prompts, blocks, allseq)
    assert dec.bucket(len(ids), 10).bm == 128
    dmeta = _decode_meta(cfg, prompts, blocks, allseq)
    b = dec.bucket(10, 10)
    b.load(dmeta, tok.numpy())
    dec.step(b, 1)
    torch.cuda.synchronize()
    lp_d, tok_d = b.logprobs.cpu().clone(), b.tokens.cpu().clone()

    w2 = DecoderWeights(cfg, device="cuda", seed=13, std=0.05, norm_std=0.1)
    both = w2.nbytes()
    w2.pack_experts(keep_unpacked=False)
    assert w2.packed_only and all(l["gate_up"] is None and l["down"] is None for l in w2.layers)
    assert w2.nbytes() >= both  # the packed image pads K to a multiple of 256
    with pytest.raises(RuntimeError):
        w2.invalidate_packed()
    dec2 = Qwen3MoeDecoder(cfg, w2, num_cache_blocks=dec.key_cache[0].shape[0])
    tok2, lp2, _, _ = _prefill(dec2, cfg, prompts, blocks, allseq)
    assert dec2.bucket(len(ids), 10).bm == 256
    assert_bitwise(lp2, lp, "prefill logprobs: packed-only model vs [E, N, K] model")
    assert torch.equal(tok2, tok)
    b2 = dec2.bucket(10, 10)
    b2.load(dmeta, tok.numpy())
    dec2.step(b2, 1)
    torch.cuda.synchronize()
    assert_bitwise(b2.logprobs.cpu(), lp_d, "decode logprobs: packed-only model vs [E, N, K] model")
    assert torch.equal(b2.tokens.cpu(), tok_d)


def test_decode_on_packed_expert_weights_keeps_every_bit():
    # the same decode step with the experts streamed from their fragment-order copies: eager and in a graph
    cfg, w, dec, prompts, blocks = _setup(num_seqs=6, seed=9)
    allseq = list(range(6))
    tok, _, _, _ = _prefill(dec, cfg, prompts, blocks, allseq)
    dmeta = _decode_meta(cfg, prompts, blocks, allseq)
    b = dec.bucket(6, 6)
    b.load(dmeta, tok.numpy())
    dec.step(b, 1)
    torch.cuda.synchronize()
    lp0, tok0 = b.logprobs.cpu().clone(), b.tokens.cpu().clone()
    w.pack_experts()
    b.load(dmeta, tok.numpy())
    dec.step(b, 1)
    torch.cuda.synchronize()
    assert_bitwise(b.logprobs.cpu(), lp0, "decode logprobs: packed vs [E, N, K] expert weights")
    assert torch.equal(b.tokens.cpu(), tok0)
    b.load(dmeta, tok.numpy())
    graph = dec.capture(b, 1)
    for _ in range(2):
        b.logprobs.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert_bitwise(b.logprobs.cpu(), lp0, "graph replay on packed expert weights")
    # a weight update the copies know nothing about: stale until invalidated, then the new weights decide
    with torch.no_grad():
        w.layers[0]["down"].mul_(-0.5)
    b.load(dmeta, tok.numpy())
    dec.step(b, 1)
    torch.cuda.synchronize()
    assert_bitwise(b.logprobs.cpu(), lp0, "the copies are not tracked: an eager step still reads the old ones")
    w.invalidate_packed()
    b.load(dmeta, tok.numpy())
    dec.step(b, 1)
    torch.cuda.synchronize()
    lp_new = b.logprobs.cpu().clone()
    assert not torch.equal(lp_new, lp0), "after invalidate_packed the updated weights are read"
    w.pack_experts()
    b.load(dmeta, tok.numpy())
    dec.step(b, 1)
    torch.cuda.synchronize()
    assert_bitwise(b.logprobs.cpu(), lp_new, "repacked copies of the updated weights")
