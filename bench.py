#!/usr/bin/env python3
"""Headline benchmark: decode tok/s of a Qwen3-30B-A3B-shaped decoder at batch 256 on one MI355X.

Workload (synthetic, seeded): 48 layers, hidden 2048, 32 q / 4 kv heads x 128, 128 experts top-8
(moe_intermediate 768), vocab 151936, random-init bf16 weights ~N(0, 0.02); 256 sequences with prompt
lengths uniform in [256, 2048] of random token ids, paged KV (page 16, block tables from a random
permutation of the pool). The prompts are prefilled with this library's own kernels, then ONE decode
step (256 tokens, 256 sequences, greedy token + fp32 logprob) is captured in a HIP graph and
replayed: warm-up W times, then exactly K timed replays.

Prints one JSON line: whole-job tok/s, the roofline of the dominant kernel (MoE gate/up grouped
GEMM, HBM bound) measured with HIP events, per-kernel GB/s of the other memory-bound kernels, the
logprob bit drift between batch 256 and batch 1 for every request, an advancing decode loop (per-step host
metadata + one host-to-device copy + graph replay + sampled tokens fed back) beside the replay figure, the
reference's other configurations (op chain, decode attention, chunked prefill, fused MoE) and the prefill
q/k/v GEMM against their HBM / MFMA rooflines, and the CPU oracle timed on the host cores for a bounded
sample (one decoder layer + lm_head at batch 256, scaled to 48 layers).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--layers", type=int, default=48, help="fewer layers = a smoke run, flagged as such in the output")
    ap.add_argument("--min-prompt", type=int, default=256)
    ap.add_argument("--max-prompt", type=int, default=2048)
    ap.add_argument("--drift-requests", type=int, default=256, help="requests re-run at batch 1 for the bit-drift check")
    ap.add_argument("--loop-steps", type=int, default=20,
                    help="steps of the advancing decode loop (host metadata + copy + replay + token feedback); 0 = skip")
    ap.add_argument("--no-configs", action="store_true", help="skip the reference's other configurations (C1-C4, prefill GEMM)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-dropin", action="store_true", help="skip the HuggingFace drop-in decode step (dropin_ms_per_step keys)")
    ap.add_argument("--no-packed-experts", action="store_true",
                    help="every step reads the [E, N, K] expert tensors instead of their fragment-order copies")
    ap.add_argument("--keep-unpacked-experts", action="store_true",
                    help="keep the [E, N, K] expert tensors beside their fragment-order copies (a second copy of the "
                         "expert weights; the default holds the fragment-order copies only)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--seed", type=int, default=5)
    ap.add_argument("--cpu-configs", action="store_true",
                    help="time the CPU oracle on the reference's other configurations (op chain, decode attention, "
                         "chunked prefill, fused MoE) instead of running the GPU benchmark; prints one JSON line")
    return ap.parse_args()


def cpu_configs(seed):
    """CPU legs of the reference configurations C1 - C4: the oracle (torch CPU restatement) timed on this
    host's cores at the full shapes (chunked prefill: 2 of the 16 sequences, scaled by the work)."""
    import numpy as np
    import torch

    from oracle import attention as OA
    from oracle import moe as OM
    from oracle.row_ops import hf_rms_norm_ref, log_softmax_ref, matmul_ref

    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(seed)

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

    def timed(fn, reps=2):
        fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return (time.perf_counter() - t0) / reps

    res = {"cores": cores, "kind": "port"}
    # C1: RMSNorm -> lm_head -> fp32 log_softmax, H = 2048, V = 151936
    H, V = 2048, 151936
    wl, wn = rnd(V, H, std=0.02), (1 + 0.02 * torch.randn(H, generator=g)).to(torch.bfloat16)
    for M in (1, 64):
        x = rnd(M, H)
        res[f"C1 op chain M={M} (s)"] = round(timed(lambda: log_softmax_ref(matmul_ref(hf_rms_norm_ref(x, wn), wl.t()).float())), 4)
    del wl
    # C2: decode attention, 64 sequences, context 128..4096, Hq = 16, Hkv = 8, D = 128, page 16
    rng = np.random.default_rng(2)
    L = rng.integers(128, 4097, size=64)
    k_seqs = [rnd(int(n), 8, 128) for n in L]
    v_seqs = [rnd(int(n), 8, 128) for n in L]
    kc, vc, table = OA.make_paged_kv_cache(k_seqs, v_seqs, 16)
    q = rnd(64, 16, 128)
    cu = torch.arange(65, dtype=torch.int32)
    used = torch.tensor(L, dtype=torch.int32)
    res["C2 decode attention B=64 (s)"] = round(timed(lambda: OA.paged_attention_ref(q, kc, vc, cu, used, table, 128 ** -0.5)), 4)
    del kc, vc, k_seqs, v_seqs
    # C3: chunked prefill, 512-token chunks on prefixes 0..8192, Hq = 32, Hkv = 8: 2 of 16 sequences
    prefix = np.random.default_rng(3).integers(0, 8193, size=16)
    work = lambda P: 512 * P + 512 * 513 // 2  # noqa: E731
    sub = [int(prefix[0]), int(prefix[1])]
    qs = [rnd(512, 32, 128) for _ in sub]
    ks = [rnd(P + 512, 8, 128) for P in sub]
    vs = [rnd(P + 512, 8, 128) for P in sub]
    t = timed(lambda: [OA.eager_attention(a, b, c, 128 ** -0.5) for a, b, c in zip(qs, ks, vs)], reps=1)
    res["C3 chunked prefill 16 x 512 (s, scaled from 2 sequences)"] = round(t * sum(work(int(P)) for P in prefix) / sum(work(P) for P in sub), 3)
    # C4: fused MoE block, H = 2048, I = 768, 128 experts, top-8
    E, k, I = 128, 8, 768
    gw, uw, dw = rnd(E, I, H, std=0.02), rnd(E, I, H, std=0.02), rnd(E, H, I, std=0.02)
    for T in (1, 64, 256):
        x = rnd(T, H)
        w, idx = OM.router_ref(torch.randn(T, E, generator=g), k)
        res[f"C4 fused MoE T={T} (s)"] = round(timed(lambda: OM.fused_moe_ref(x, w, idx, gw, uw, dw), reps=1), 4)
    print(json.dumps({"cpu_configs": res}), flush=True)


def build_workload(layers=48, batch=256, seed=5, min_prompt=256, max_prompt=2048, grow=1, packed=True, log=True,
                   keep_unpacked=False):
    """The headline workload: random-init weights, ``batch`` prompts of random ids prefilled with the library's own
    kernels into a paged cache (page 16, block tables from a random permutation of the pool, room for ``grow``
    more tokens per sequence), and the metadata of the decode step that follows."""
    import types

    import torch

    from vexact_amd.decoder import DecoderWeights, Qwen3MoeDecoder, build_step_metadata, qwen3_30b_a3b

    dev = "cuda"
    say = (lambda m: print(m, file=sys.stderr, flush=True)) if log else (lambda m: None)
    cfg = qwen3_30b_a3b()
    cfg.num_layers = layers
    B = batch
    rng = np.random.default_rng(seed)
    prompt_lens = rng.integers(min_prompt, max_prompt + 1, size=B)
    prompts = [rng.integers(0, cfg.vocab_size, size=int(n)) for n in prompt_lens]
    pages = [(int(n) + grow + cfg.page_size - 1) // cfg.page_size for n in prompt_lens]
    pool = sum(pages) + 64
    perm = rng.permutation(pool)
    blocks, o = [], 0
    for p in pages:
        blocks.append(perm[o : o + p].tolist())
        o += p
    max_blocks = (cfg.max_model_len + cfg.page_size - 1) // cfg.page_size

    t0 = time.time()
    w = DecoderWeights(cfg, device=dev, seed=seed)
    # Expert weights in fragment order (made once per weight update): decode streams them, and the 256-row expert
    # tiles of the prefill chunks read them too, so the [E, N, K] tensors are freed unless asked for.
    if packed:
        w.pack_experts(keep_unpacked=keep_unpacked)
    dec = Qwen3MoeDecoder(cfg, w, num_cache_blocks=pool, device=dev)
    torch.cuda.synchronize()
    say(f"[bench] weights {w.nbytes() / 1e9:.1f} GB"
        f"{' + a second copy of the experts in fragment order' if packed and keep_unpacked else ''}, KV pool {pool} pages "
        f"({2 * cfg.num_layers * dec.key_cache[0].numel() * 2 / 1e9:.1f} GB), init {time.time() - t0:.1f}s")

    # ---- prefill with the library's own kernels, several sequences per pass
    t0 = time.time()
    PT, PB = 8192, 16
    pb = dec.bucket(PT, PB)
    first_tokens = np.zeros(B, dtype=np.int64)
    s = 0
    while s < B:
        grp, tot = [], 0
        while s < B and len(grp) < PB and tot + len(prompts[s]) <= PT:
            grp.append(s)
            tot += len(prompts[s])
            s += 1
        reqs = [dict(num_computed_tokens=len(prompts[i]), tokens_this_step=len(prompts[i]), block_ids=blocks[i]) for i in grp]
        _, _, max_q = pb.load_requests(reqs, np.concatenate([prompts[i] for i in grp]), cfg.page_size)
        dec.step(pb, max_q)
        first_tokens[grp] = pb.tokens[: len(grp)].cpu().numpy()
    torch.cuda.synchronize()
    say(f"[bench] prefill of {int(prompt_lens.sum())} tokens: {time.time() - t0:.1f}s")
    del dec.buffers[(PT, PB)]
    del pb
    torch.cuda.empty_cache()

    ctx = [int(n) + 1 for n in prompt_lens]
    reqs = [dict(num_computed_tokens=ctx[i], tokens_this_step=1, block_ids=blocks[i]) for i in range(B)]
    dmeta = build_step_metadata(reqs, cfg.page_size, max_blocks)
    return types.SimpleNamespace(cfg=cfg, w=w, dec=dec, B=B, prompts=prompts, prompt_lens=prompt_lens, blocks=blocks,
                                 ctx=ctx, reqs=reqs, dmeta=dmeta, first_tokens=first_tokens, max_blocks=max_blocks, pool=pool)


def drift_check(wl, lp_batch, tok_batch, n):
    """Re-run ``n`` of the workload's requests alone (batch 1, eager) and count the bits in which the logprob
    differs from the batched step's (64 more for a different token). Returns (bits, requests checked)."""
    import torch

    from vexact_amd.decoder import build_step_metadata

    bits, checked = 0, 0
    b1 = wl.dec.bucket(1, 1)
    for i in range(min(n, wl.B)):
        r = (i * 37) % wl.B
        m1 = build_step_metadata([wl.reqs[r]], wl.cfg.page_size, wl.max_blocks)
        b1.load(m1, wl.first_tokens[r : r + 1])
        wl.dec.step(b1, 1)
        torch.cuda.synchronize()
        a = b1.logprobs.cpu().view(torch.int32)
        bb = lp_batch[r : r + 1].view(torch.int32)
        bits += bin((int(a[0]) ^ int(bb[0])) & 0xFFFFFFFF).count("1") + (0 if int(b1.tokens[0]) == int(tok_batch[r]) else 64)
        checked += 1
    return bits, checked


def main():
    args = parse()
    if args.cpu_configs:
        cpu_configs(args.seed)
        return
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (all pipeline stages collapsed onto one MI355X); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)
    out = headline(args)  # everything the built-in decoder holds on the GPU dies with that call's frame
    if not args.no_dropin and out["config"]["full_model"]:
        # What a caller of the reference gets by switching imports (a HuggingFace Qwen3MoeForCausalLM through the
        # registered attention function, the patched modules and batch-invariant mode): the same decode step, captured
        # in a graph. It needs the memory the built-in decoder held.
        import gc

        import torch
        gc.collect()
        torch.cuda.empty_cache()
        out.update(dropin_step(args.batch))
    print(json.dumps(out), flush=True)


def headline(args):
    import torch

    from vexact_amd import _build, _lib, ops
    from vexact_amd.decoder import decode_bytes_per_step

    if not os.path.exists(_build.LIB_PATH):
        _build.build()
    _lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda"
    torch.cuda.set_device(0)

    wl = build_workload(args.layers, args.batch, args.seed, args.min_prompt, args.max_prompt,
                        grow=1 + max(0, args.loop_steps), packed=not args.no_packed_experts,
                        keep_unpacked=args.keep_unpacked_experts)
    cfg, w, dec, B = wl.cfg, wl.w, wl.dec, wl.B
    blocks, ctx, reqs, dmeta, first_tokens, max_blocks = wl.blocks, wl.ctx, wl.reqs, wl.dmeta, wl.first_tokens, wl.max_blocks
    E, k, I, H = cfg.num_experts, cfg.top_k, cfg.moe_intermediate, cfg.hidden_size

    def moe_gate_up(li, lw, r):
        if w.packed is not None:
            pg = w.packed[li][0]
            return ops.moe_gemm_packed(db.h, pg.rows(0, I), r, w2=pg.rows(I, 2 * I), row_src=r.sorted_token,
                                       row_scale=db.topk_w, row_scale_idx=r.sorted_flat, out=db.hw)
        gu = lw["gate_up"]
        return ops.moe_gemm(db.h, gu[:, :I, :], r, w2=gu[:, I:, :], row_src=r.sorted_token, row_scale=db.topk_w,
                            row_scale_idx=r.sorted_flat, out=db.hw)

    def moe_down(li, lw, r):
        if w.packed is not None:
            return ops.moe_gemm_packed(db.hw, w.packed[li][1], r, out=db.eo)
        return ops.moe_gemm(db.hw, lw["down"], r, out=db.eo)

    # ---- the decode step: 256 tokens, 256 sequences, captured in a HIP graph
    db = dec.bucket(B, B)
    db.load(dmeta, first_tokens)
    graph = dec.capture(db, 1)
    for _ in range(args.warmup):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graph.replay()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    tok_s = B * args.steps / dt
    lp_graph = db.logprobs.cpu().clone()
    tok_graph = db.tokens.cpu().clone()

    # ---- logprob bit drift: the same requests at batch 1 (eager)
    t0 = time.time()
    drift_bits, checked = drift_check(wl, lp_graph, tok_graph, args.drift_requests)
    print(f"[bench] drift check of {checked} requests at batch 1: {time.time() - t0:.1f}s, {drift_bits} bits", file=sys.stderr, flush=True)

    # ---- an advancing decode loop: what a serving step pays around the graph (inferencer.py:124-191, 193-349):
    # native step metadata into the pinned staging buffer, ONE host-to-device copy, graph replay, sampled
    # tokens back to the host (the scheduler appends them to the requests) and in as the next input ids,
    # every context one token longer
    loop = None
    if args.loop_steps > 0:
        lreqs = [dict(num_computed_tokens=ctx[i], tokens_this_step=1, block_ids=np.asarray(blocks[i], np.int32)) for i in range(B)]
        toks = first_tokens.copy()
        host_s = 0.0
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.loop_steps):
            h0 = time.perf_counter()
            db.load_requests(lreqs, toks, cfg.page_size)
            host_s += time.perf_counter() - h0
            graph.replay()
            toks = db.tokens.cpu().numpy()  # waits for the step
            h0 = time.perf_counter()
            for r_ in lreqs:
                r_["num_computed_tokens"] += 1
            host_s += time.perf_counter() - h0
        dt_loop = time.perf_counter() - t0
        loop = {"decode_loop_tok_s": round(B * args.loop_steps / dt_loop, 1), "loop_steps": args.loop_steps,
                "loop_ms_per_step": round(dt_loop / args.loop_steps * 1e3, 3),
                "host_ms_per_step": round(host_s / args.loop_steps * 1e3, 3),
                "what": "per step: vx_host_step_metadata into pinned staging + one H2D copy, graph replay, tokens D2H and "
                        "fed back as the next input ids, contexts growing by one"}

    # ---- per-kernel timing with HIP events on the launch stream (eager pass over all layers)
    ev = lambda: torch.cuda.Event(enable_timing=True)  # noqa: E731
    names = ("moe_gate_up", "moe_down", "attn_decode", "qkv_gemm", "o_gemm")
    times = {n: [] for n in names}
    reps = 2
    scale = cfg.head_dim ** -0.5
    experts_hit = []
    for rep in range(reps + 1):
        pend = []
        db.load(dmeta, first_tokens)
        ops.embedding(w.embed, db.input_ids, out=db.x)
        ops.rms_norm(db.x, w.layers[0]["in_norm"], cfg.rms_eps, hf_two_rounding=True, out=db.h)
        for li, lw in enumerate(w.layers):
            def timed(name, fn):
                a, b_ = ev(), ev()
                a.record()
                fn()
                b_.record()
                pend.append((name, a, b_))
            timed("qkv_gemm", lambda: ops.gemm_nt(db.h, lw["qkv"], out=db.qkv))
            ops.qk_norm_rope_store(db.qkv, lw["q_norm"], lw["k_norm"], dec.cos, dec.sin, db.positions, db.slot_mapping,
                                   db.q, dec.key_cache[li], dec.value_cache[li], cfg.num_heads, cfg.num_kv_heads,
                                   cfg.head_dim, cfg.rms_eps)
            timed("attn_decode", lambda: ops.paged_attention(db.q, dec.key_cache[li], dec.value_cache[li], db.query_start_loc,
                                                             db.context_lens, db.block_tables, scale, 1, out=db.attn,
                                                             workspace=db.attn_ws, seq_order=db.seq_order))
            timed("o_gemm", lambda: ops.gemm_nt(db.attn.view(B, -1), lw["o"], out=db.o))
            ops.rms_norm(db.o, lw["post_norm"], cfg.rms_eps, hf_two_rounding=True, residual=db.x, sum_out=db.x, out=db.h)
            ops.gemm_nt(db.h, lw["router"], out=db.router_logits)
            dec._router(db)
            r = ops.moe_route(db.topk_idx, E, bm=db.bm, buffers=db.route_ints)
            if rep == 0:
                experts_hit.append(int((r.splits > 0).sum()))
            timed("moe_gate_up", lambda: moe_gate_up(li, lw, r))
            timed("moe_down", lambda: moe_down(li, lw, r))
            nxt = w.layers[li + 1]["in_norm"] if li + 1 < cfg.num_layers else w.final_norm
            ops.moe_gather(db.eo, r.scatter_index, residual=db.x, out=db.x)
            ops.rms_norm(db.x, nxt, cfg.rms_eps, hf_two_rounding=True, out=db.h)
        torch.cuda.synchronize()
        if rep > 0:  # first pass is a warm-up
            for name, a, b_ in pend:
                times[name].append(a.elapsed_time(b_) * 1e-3)
    avg = {n: float(np.mean(v)) for n, v in times.items()}
    # The dominant kernel once more, as it runs in the decode graph: back to back in a captured graph (one
    # launch per layer's weights, the last layer's routing), HIP events around each replay. Eager launches
    # above carry a few microseconds of launch and event overhead per kernel; this figure is the one that
    # matches a kernel trace of the graph.
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())

    def gate_up_all_layers():
        for li_, lw_ in enumerate(w.layers):
            moe_gate_up(li_, lw_, r)

    with torch.cuda.stream(side):
        gate_up_all_layers()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    kgraph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(kgraph):
        gate_up_all_layers()
    kgraph.replay()
    torch.cuda.synchronize()
    in_graph = []
    for _ in range(5):
        a, b_ = ev(), ev()
        a.record()
        kgraph.replay()
        b_.record()
        torch.cuda.synchronize()
        in_graph.append(a.elapsed_time(b_) * 1e-3 / len(w.layers))
    avg_in_graph = float(np.mean(in_graph))
    U = float(np.mean(experts_hit))
    sumL = int(sum(ctx))
    kbytes = {
        "moe_gate_up": U * 2 * I * H * 2 + B * H * 2 + B * k * I * 2 + B * k * 6,
        "moe_down": U * H * I * 2 + B * k * I * 2 + B * k * H * 2,
        "attn_decode": sumL * 2 * cfg.num_kv_heads * cfg.head_dim * 2 + 2 * B * cfg.num_heads * cfg.head_dim * 2
        + sum((c + cfg.page_size - 1) // cfg.page_size for c in ctx) * 4,
        "qkv_gemm": 2 * (cfg.qkv_dim * H + B * H + B * cfg.qkv_dim),
        "o_gemm": 2 * (H * cfg.num_heads * cfg.head_dim + B * cfg.num_heads * cfg.head_dim + B * H),
    }
    kernels = {n: {"avg_us": round(avg[n] * 1e6, 1), "bytes": int(kbytes[n]), "GBps": round(kbytes[n] / avg[n] / 1e9, 1),
                   "frac_hbm": round(kbytes[n] / avg[n] / 1e9 / HBM_PEAK_GBS, 4)} for n in names}
    dom = "moe_gate_up"
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        try:
            traffic = json.load(open(tpath)).get(dom if w.packed is not None else dom + "_unpacked")
        except Exception:
            traffic = None
    kernels[dom]["in_graph_avg_us"] = round(avg_in_graph * 1e6, 1)
    achieved = kbytes[dom] / avg_in_graph / 1e9
    roofline = {"bound": "hbm", "kernel": "gemm_stream_kernel<2, SWIGLU, grouped%s> (MoE gate/up)" % (", packed" if w.packed is not None else ""),
                "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                "timing": "HIP events around graph replays of 48 back-to-back launches (one per layer's weights)"}

    step_bytes = decode_bytes_per_step(cfg, ctx, experts_hit_per_layer=U)
    out = {
        "metric": "decode tok/s Qwen3-30B-A3B bs=256 on 1 GPU",
        "value": round(tok_s, 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"Qwen3-30B-A3B-shaped decoder ({cfg.num_layers} layers, 128 experts top-8, vocab 151936), "
                               f"hipGraph decode step, batch {B}, prompts U[{args.min_prompt},{args.max_prompt}], paged KV page 16",
                   "batch": B, "sum_context": sumL, "full_model": cfg.num_layers == 48 and B == 256},
        "weights_gb": round(w.nbytes() / 1e9, 1),
        "expert_weight_copies": 1 if (w.packed is None or w.packed_only) else 2,
        "step_hbm_bytes": int(step_bytes["total"]),
        "step_frac_of_hbm_roofline": round(step_bytes["total"] / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "logprob_drift_bits_b256_vs_b1": drift_bits,
        "drift_requests_checked": checked,
        "roofline": roofline,
        "kernels": kernels,
    }

    if loop is not None:
        out.update(loop)
    if not args.no_configs:
        out["configs"], out["roofline_mfma"] = other_configs()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, w, dec, dmeta, first_tokens, B, args.cpu_seconds)
    return out


def dropin_step(batch):
    """``dropin_ms_per_step`` (the reference's cache layout, graph captured with ``max_seqlen_q = 1``),
    ``dropin_ms_per_step_reference_capture`` (captured the way the reference's CudaGraphManager does, with
    ``max_seqlen_q`` = the bucket's tokens) and ``dropin_ms_per_step_head_major`` (``KVCacheStore(head_major=True)``)."""
    import kernel_bench

    rows = kernel_bench.dropin_decode(kernel_bench.parse(["--what", "dropin", "--batch", str(batch)]), quiet=True)
    out = {"dropin": rows}
    for r in rows:
        key = "dropin_ms_per_step" + ("_head_major" if r["head_major"] else "_reference_capture" if r["max_seqlen_q"] != 1 else "")
        out[key] = r["ms_per_step"]
    return out


def other_configs():
    """The reference's other benchmark configurations at their own shapes, graph-replayed and timed with HIP
    events (kernel_bench.py): C1 op chain at M = 1 / 7 / 64, C2 decode attention, C3 chunked prefill attention,
    C4 fused MoE block at T = 1 / 64 / 256 / 4096, the q/k/v projection of an 8192-token prefill chunk, and the
    training side's kernels (packed attention forward / backward, the MoE backward products at 8192 tokens).
    Each line carries its algorithmic bytes or flops and the fraction of the HBM / bf16 MFMA peak."""
    import kernel_bench

    res = kernel_bench.run(kernel_bench.parse(["--what", "configs,mfma,train", "--batch", "256", "--layers", "2", "--reps", "3"]),
                           quiet=True)
    mfma = [r for r in res if r["bound"] == "mfma"]
    return res, mfma


def cpu_baseline(cfg, w, dec, dmeta, first_tokens, B, budget_s):
    """The CPU oracle (torch CPU restatement of the reference's formulas) on this host's cores: one
    decoder layer + lm_head at the bench batch, scaled to all layers."""
    import torch

    from oracle import decoder as OD
    from oracle.row_ops import hf_rms_norm_ref, logprobs_ref, matmul_ref
    from vexact_amd import ops
    # threads: the harness gives a one-GPU job 16 host cores (OMP_NUM_THREADS), whatever os.cpu_count() shows
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    torch.set_num_threads(cores)
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    lw = {k_: v.cpu() for k_, v in w.layers[0].items() if v is not None}
    if w.packed_only:  # the oracle wants [E, N, K]
        lw["gate_up"] = ops.unpack_expert_weights(w.packed[0][0]).cpu()
        lw["down"] = ops.unpack_expert_weights(w.packed[0][1]).cpu()
    kc, vc = dec.key_cache[0].cpu().contiguous(), dec.value_cache[0].cpu().contiguous()
    cos, sin = OD.rope_tables_ref(cfg.head_dim, cfg.rope_theta, cfg.max_model_len)
    x = w.embed[torch.as_tensor(first_tokens).to(w.embed.device)].cpu()
    pos = torch.as_tensor(dmeta["positions"]).long()
    lm_head, fnorm = w.lm_head.cpu(), w.final_norm.cpu()
    t_layer, t_head, n = 0.0, 0.0, 0
    t_start = time.perf_counter()
    while True:
        t0 = time.perf_counter()
        y = OD.layer_ref(cfg, lw, x, pos, dmeta, kc, vc, cos, sin)
        t1 = time.perf_counter()
        logits = matmul_ref(hf_rms_norm_ref(y, fnorm, cfg.rms_eps), lm_head.t())
        tok = logits.float().argmax(-1)
        logprobs_ref(logits.float(), tok)
        t2 = time.perf_counter()
        t_layer += t1 - t0
        t_head += t2 - t1
        n += 1
        if time.perf_counter() - t_start > budget_s or n >= 5:
            break
    step = cfg.num_layers * t_layer / n + t_head / n
    return {"value": round(B / step, 3), "unit": "tok/s", "cores": cores, "kind": "port", "cpu_model": model,
            "host_cpus": os.cpu_count(),
            "sample": f"1 of {cfg.num_layers} decoder layers + lm_head at batch {B}, {n} repeats "
                      f"({t_layer / n:.2f}s per layer, {t_head / n:.2f}s head), scaled to {cfg.num_layers} layers"}


if __name__ == "__main__":
    main()
