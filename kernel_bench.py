#!/usr/bin/env python3
"""Per-kernel micro-benchmarks at the headline shapes (Qwen3-30B-A3B decode, batch 256).

Each kernel is launched once per "layer" on its own copy of the weights / KV cache (so nothing is
served from the caches), the loop over layers is captured in a HIP graph to keep host launch cost
out, and the replay is timed with events. Prints time, algorithmic bytes (or flops) and the
fraction of the MI355X peak. ``--nograph`` launches eagerly once and times nothing: that is the form
to run under ``rocprofv3 --pmc``.

    python kernel_bench.py --what moe,attn,gemm,small,prefill,dense,train,sampler,other,configs,mfma,copy,dropin,trainlayer
"""

from __future__ import annotations

import argparse
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from vexact_amd import _lib, ops  # noqa: E402

HBM_PEAK = 8.0e12
MFMA_PEAK = 2.5e15


def parse(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--what", default="moe,attn,gemm,small")
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--layers", type=int, default=6, help="independent weight / cache copies to rotate over")
    ap.add_argument("--reps", type=int, default=5, help="timed graph replays (at least; see --min-ms)")
    ap.add_argument("--settle-ms", type=float, default=40.0, help="untimed replays before the timed ones")
    ap.add_argument("--min-ms", type=float, default=10.0, help="the timed replays cover at least this long")
    ap.add_argument("--kv-layout", default="fused", choices=("head", "token", "fused"),
                    help="physical KV cache layout: fused = [blocks, Hkv, 2, page, D] (what the decoder allocates), head = [blocks, Hkv, page, D] per tensor, token = [blocks, page, Hkv, D]")
    ap.add_argument("--page", type=int, default=16, help="KV cache page size (keys)")
    ap.add_argument("--nograph", action="store_true", help="eager launches only, no timing (for rocprofv3 --pmc)")
    ap.add_argument("--dropin-head-major", action="store_true",
                    help="section dropin: KVCacheStore(head_major=True) instead of the reference's cache layout")
    return ap.parse_args(argv)


def run(a, quiet: bool = False) -> list:
    """Run the sections named in ``a.what``; returns one dict per reported line (name, us, bytes or flops,
    achieved rate, fraction of the MI355X peak)."""
    dev = "cuda"
    results = []
    B, NL = a.batch, a.layers
    H, I, E, k = 2048, 768, 128, 8
    g = torch.Generator(device=dev).manual_seed(0)

    def rnd(*s, std=0.02):
        t = torch.empty(s, dtype=torch.bfloat16, device=dev)
        t.normal_(0, std, generator=g)
        return t

    def timeit(fn, n_layers=NL):
        """Seconds per call of ``fn`` inside a captured graph of ``n_layers`` calls, at steady clocks: the graph is
        replayed for ``--settle-ms`` first (after an idle spell this machine runs heavy kernels up to 25 % slower for
        the first ~20 ms), then ``--reps`` replays, and more until they cover ``--min-ms``, are timed as one span."""
        for li in range(n_layers):
            fn(li)
        torch.cuda.synchronize()
        if a.nograph:
            return None
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for li in range(n_layers):
                fn(li)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        one = max(e0.elapsed_time(e1), 1e-3)  # ms per replay, first estimate
        for _ in range(min(2000, int(a.settle_ms / one) + 1)):
            graph.replay()
        reps = max(a.reps, min(2000, int(a.min_ms / one) + 1))
        e0.record()
        for _ in range(reps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / (reps * n_layers)

    def report(name, t, nbytes=None, flops=None):
        say = (lambda *x, **k: None) if quiet else print
        if t is None:
            say(f"{name:34s} launched", flush=True)
        elif flops is not None:
            results.append({"name": name, "us": round(t * 1e6, 1), "flops": int(flops), "bound": "mfma",
                            "TFLOPs": round(flops / t / 1e12, 1), "frac": round(flops / t / MFMA_PEAK, 4)})
            say(f"{name:34s} {t * 1e6:9.1f} us  {flops / t / 1e12:8.1f} TFLOP/s  ({flops / t / MFMA_PEAK * 100:5.1f}% of 2.5 PFLOP/s)", flush=True)
        else:
            results.append({"name": name, "us": round(t * 1e6, 1), "bytes": int(nbytes), "bound": "hbm",
                            "GBps": round(nbytes / t / 1e9, 1), "frac": round(nbytes / t / HBM_PEAK, 4)})
            say(f"{name:34s} {t * 1e6:9.1f} us  {nbytes / t / 1e9:8.1f} GB/s  ({nbytes / t / HBM_PEAK * 100:5.1f}% of 8 TB/s)  {nbytes / 1e6:.1f} MB", flush=True)

    what = a.what.split(",") if isinstance(a.what, str) else list(a.what)
    if "sampler" in what:
        V = 151936
        lg = (torch.randn(B, V, generator=g, device=dev) * 2.5).to(torch.bfloat16)
        seeds = torch.arange(B, dtype=torch.int64, device=dev) + 1234
        pos = torch.arange(B, dtype=torch.int64, device=dev) + 1000
        out = torch.empty(B, dtype=torch.int64, device=dev)
        for name, top_k, top_p in (("plain", None, 1.0), ("top-p 0.9", None, 0.9), ("top-k 50", 50, 1.0), ("top-k 50 + top-p 0.9", 50, 0.9)):
            report(f"sampler {name} (B={B}, V={V})",
                   timeit(lambda li: ops.sample_tokens(lg, 0.8, top_k, top_p, seeds, pos, out=out), n_layers=4), B * V * 2)
        report("greedy argmax + logprob", timeit(lambda li: ops.logprobs(lg, None, return_tokens=True), n_layers=4), B * V * 2)
    if "moe" in what:
        x = rnd(B, H, std=1.0)
        logits = torch.randn(B, E, generator=g, device=dev)
        w, idx = ops.router_topk(logits, k, index_dtype=torch.int32)
        r = ops.moe_route(idx, E, bm=ops.moe_tile_rows(B))
        U = int((r.splits > 0).sum())
        gu = [rnd(E, 2 * I, H + 64)[..., :H] for _ in range(NL)]  # 128 bytes of row padding, as the decoder allocates them
        dn = [rnd(E, H, I) for _ in range(NL)]
        hw = torch.empty(B * k, I, dtype=torch.bfloat16, device=dev)
        eo = torch.empty(B * k, H, dtype=torch.bfloat16, device=dev)
        y = torch.empty(B, H, dtype=torch.bfloat16, device=dev)
        report(f"moe gate/up (B={B}, {U} experts)",
               timeit(lambda li: ops.moe_gemm(x, gu[li][:, :I, :], r, w2=gu[li][:, I:, :], row_src=r.sorted_token,
                                              row_scale=w, row_scale_idx=r.sorted_flat, out=hw)),
               U * 2 * I * H * 2 + B * H * 2 + B * k * I * 2 + B * k * 6)
        report("moe down", timeit(lambda li: ops.moe_gemm(hw, dn[li], r, out=eo)), U * H * I * 2 + B * k * I * 2 + B * k * H * 2)
        pgu = [ops.pack_expert_weights(t) for t in gu]  # fragment-order copies, as the decoder streams them
        pdn = [ops.pack_expert_weights(t) for t in dn]
        report(f"moe gate/up, packed weights",
               timeit(lambda li: ops.moe_gemm_packed(x, pgu[li].rows(0, I), r, w2=pgu[li].rows(I, 2 * I), row_src=r.sorted_token,
                                                     row_scale=w, row_scale_idx=r.sorted_flat, out=hw)),
               U * 2 * I * H * 2 + B * H * 2 + B * k * I * 2 + B * k * 6)
        report("moe down, packed weights", timeit(lambda li: ops.moe_gemm_packed(hw, pdn[li], r, out=eo)),
               U * H * I * 2 + B * k * I * 2 + B * k * H * 2)
        report("moe route", timeit(lambda li: ops.moe_route(idx, E, bm=32)), B * k * 16)
        report("moe gather + residual", timeit(lambda li: ops.moe_gather(eo, r.scatter_index, residual=x, out=y)),
               B * k * H * 2 + 2 * B * H * 2)
        lb = logits.to(torch.bfloat16)
        report("router top-k (bf16 logits)", timeit(lambda li: ops.router_topk(lb, k, index_dtype=torch.int32)), B * E * 2)
    if "attn" in what:
        Hq, Hkv, D, page = 32, 4, 128, a.page
        rng = np.random.default_rng(5)
        L = rng.integers(257, 2050, size=B)
        pages = [(int(n) + page - 1) // page for n in L]
        pool = sum(pages) + 64
        perm = rng.permutation(pool)
        maxb = 4096 // page
        bt = np.full((B, maxb), -1, np.int32)
        o = 0
        for s, p in enumerate(pages):
            bt[s, :p] = perm[o : o + p]
            o += p
        if a.kv_layout == "fused":  # one kv head's K page and V page adjacent: [blocks, Hkv, 2, page, D]
            kv = [rnd(pool, Hkv, 2, page, D, std=1.0) for _ in range(NL)]
            kc = [t[:, :, 0].permute(0, 2, 1, 3) for t in kv]
            vc = [t[:, :, 1].permute(0, 2, 1, 3) for t in kv]
        elif a.kv_layout == "head":
            kc = [rnd(pool, Hkv, page, D, std=1.0).permute(0, 2, 1, 3) for _ in range(NL)]
            vc = [rnd(pool, Hkv, page, D, std=1.0).permute(0, 2, 1, 3) for _ in range(NL)]
        else:
            kc = [rnd(pool, page, Hkv, D, std=1.0) for _ in range(NL)]
            vc = [rnd(pool, page, Hkv, D, std=1.0) for _ in range(NL)]
        q = rnd(B, Hq, D, std=1.0)
        cu = torch.arange(B + 1, dtype=torch.int32, device=dev)
        used = torch.tensor(L, dtype=torch.int32, device=dev)
        order = torch.tensor(np.argsort(-L, kind="stable").astype(np.int32), device=dev)  # longest first, as the host builder emits
        btd = torch.tensor(bt, device=dev)
        out = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=dev)
        ws = torch.empty(_lib.load().vx_paged_attn_decode_workspace_bytes(B, Hq, Hkv, D, 4096), dtype=torch.uint8, device=dev)
        report(f"paged decode attention (sum L={int(L.sum())})",
               timeit(lambda li: ops.paged_attention(q, kc[li], vc[li], cu, used, btd, D**-0.5, 1, out=out, workspace=ws,
                                                     seq_order=order)),
               int(L.sum()) * 2 * Hkv * D * 2 + 2 * B * Hq * D * 2 + sum(pages) * 4)
    if "gemm" in what:
        for name, N, K in (("qkv", 5120, 2048), ("o", 2048, 4096), ("router", 128, 2048), ("lm_head", 151936, 2048)):
            nl = 2 if N > 100000 else NL
            ws_ = [rnd(N, K) for _ in range(nl)]
            xx = rnd(B, K, std=1.0)
            c = torch.empty(B, N, dtype=torch.bfloat16, device=dev)
            report(f"gemm {name} M={B} N={N} K={K}", timeit(lambda li: ops.gemm_nt(xx, ws_[li], out=c), n_layers=nl),
                   2 * (N * K + B * K + B * N))
            del ws_
    if "prefill" in what:
        for name, M, N, K in (("router", 8192, 128, 2048), ("qkv", 8192, 5120, 2048), ("o", 8192, 2048, 4096), ("lm_head", 4096, 151936, 2048),
                              ("square", 8192, 8192, 8192)):
            w_ = rnd(N, K)
            xx = rnd(M, K, std=1.0)
            c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
            report(f"prefill gemm {name} M={M} N={N} K={K}", timeit(lambda li: ops.gemm_nt(xx, w_, out=c), n_layers=2),
                   flops=2 * M * N * K)
            del w_, xx, c
    if "train" in what:
        # training-side attention on packed sequences: forward with log-sum-exp, then backward
        Hq, Hkv, D, S, Lp = 32, 4, 128, 8, 1024
        q, kk, vv = rnd(S * Lp, Hq, D, std=1.0), rnd(S * Lp, Hkv, D, std=1.0), rnd(S * Lp, Hkv, D, std=1.0)
        do = rnd(S * Lp, Hq, D, std=1.0)
        cu = torch.arange(0, (S + 1) * Lp, Lp, dtype=torch.int32, device=dev)
        fl = 4 * Hq * D * S * Lp * (Lp + 1) // 2
        report("packed attention fwd + lse 8 x 1024", timeit(lambda li: ops.packed_attention(q, kk, vv, cu, cu, D**-0.5, True, Lp, return_lse=True), n_layers=2), flops=fl)
        o, lse = ops.packed_attention(q, kk, vv, cu, cu, D**-0.5, True, Lp, return_lse=True)
        report("packed attention bwd 8 x 1024", timeit(lambda li: ops.packed_attention_backward(q, kk, vv, o, do, lse, cu, cu, D**-0.5, Lp, Lp), n_layers=2), flops=fl * 5 // 2)
        # fused-MoE backward products at the model's expert shapes, 8192 tokens (256-row expert tiles)
        T = 8192
        x = rnd(T, H, std=1.0)
        logits = torch.randn(T, E, generator=g, device=dev)
        w, idx = ops.router_topk(logits, k, index_dtype=torch.int32)
        r = ops.moe_route(idx, E, bm=256)
        gu, dn = rnd(E, 2 * I, H), rnd(E, H, I)
        dyt, dg, du = rnd(T, H, std=1.0), rnd(T * k, I, std=1.0), rnd(T * k, I, std=1.0)
        o_i = torch.empty(T * k, I, dtype=torch.bfloat16, device=dev)
        o_h = torch.empty(T * k, H, dtype=torch.bfloat16, device=dev)
        o_dn, o_g = torch.empty_like(dn), torch.empty(E, I, H, dtype=torch.bfloat16, device=dev)
        report("moe bwd dgrad down (dY Wd) T=8192", timeit(lambda li: ops.moe_gemm_nn(dyt, dn, r, a_src=r.sorted_token, out=o_i), n_layers=2),
               flops=2 * T * k * H * I)
        report("moe bwd dgrad gate+up T=8192", timeit(lambda li: ops.moe_gemm_nn(dg, gu[:, :I], r, a2=du, w2=gu[:, I:], out=o_h), n_layers=2),
               flops=2 * T * k * 2 * I * H)
        report("moe bwd wgrad down T=8192", timeit(lambda li: ops.moe_gemm_tn(dyt, dg, r.cu, E, dy_src=r.sorted_token, out=o_dn), n_layers=2),
               flops=2 * T * k * H * I)
        report("moe bwd wgrad gate T=8192", timeit(lambda li: ops.moe_gemm_tn(dg, x, r.cu, E, x_src=r.sorted_token, out=o_g), n_layers=2),
               flops=2 * T * k * H * I)
        del gu, dn, o_dn, o_g
    if "dense" in what:
        # dense SwiGLU MLP of a Qwen3-8B-shaped layer (hidden 4096, intermediate 12288): fused gate/up, then down
        Hd, Id = 4096, 12288
        wg, wu, wd = rnd(Id, Hd), rnd(Id, Hd), rnd(Hd, Id)
        for M in (256, 8192):
            xx = rnd(M, Hd, std=1.0)
            hh = torch.empty(M, Id, dtype=torch.bfloat16, device=dev)
            yy = torch.empty(M, Hd, dtype=torch.bfloat16, device=dev)
            t1 = timeit(lambda li: ops.gemm_swiglu(xx, wg, wu, out=hh), n_layers=2)
            t2 = timeit(lambda li: ops.gemm_nt(hh, wd, out=yy), n_layers=2)
            if M <= 512:
                report(f"dense swiglu gate/up M={M}", t1, 2 * Id * Hd * 2 + M * Hd * 2 + M * Id * 2)
                report(f"dense down M={M}", t2, Id * Hd * 2 + M * Hd * 2 + M * Id * 2)
            else:
                report(f"dense swiglu gate/up M={M}", t1, flops=2 * M * 2 * Id * Hd)
                report(f"dense down M={M}", t2, flops=2 * M * Id * Hd)
        del wg, wu, wd
    if "prefill" in what:
        # MoE expert GEMMs over a prefill chunk (256-row expert tiles)
        for T in (4096, 8192, 32768):
            x = rnd(T, H, std=1.0)
            logits = torch.randn(T, E, generator=g, device=dev)
            w, idx = ops.router_topk(logits, k, index_dtype=torch.int32)
            r = ops.moe_route(idx, E, bm=256)
            rows = r.tile_rows[r.tile_group >= 0]
            tiles_info = f"{int(rows.numel())} row tiles, {int((rows <= 64).sum())} of at most 64 rows, {int((rows == 256).sum())} full"
            gu = rnd(E, 2 * I, H)
            dn = rnd(E, H, I)
            hw = torch.empty(T * k, I, dtype=torch.bfloat16, device=dev)
            eo = torch.empty(T * k, H, dtype=torch.bfloat16, device=dev)
            if T >= 8192:
                report(f"prefill moe route T={T}", timeit(lambda li: ops.moe_route(idx, E, bm=256), n_layers=2), T * k * 16)
                report(f"prefill moe route T={T}, one workgroup", timeit(lambda li: ops.moe_route(idx, E, bm=256, chunked=False), n_layers=2), T * k * 16)
            report(f"prefill moe gate/up T={T} ({tiles_info})",
                   timeit(lambda li: ops.moe_gemm(x, gu[:, :I, :], r, w2=gu[:, I:, :], row_src=r.sorted_token, row_scale=w,
                                                  row_scale_idx=r.sorted_flat, out=hw), n_layers=2),
                   flops=2 * T * k * 2 * I * H)
            report(f"prefill moe down T={T}", timeit(lambda li: ops.moe_gemm(hw, dn, r, out=eo), n_layers=2),
                   flops=2 * T * k * H * I)
            del x, logits, gu, dn, hw, eo
        # q/k norm + rotary + cache store over a prefill chunk
        Hq_, Hkv_, D_, page_ = 32, 4, 128, 16
        for T in (8192,):
            qkv = rnd(T, (Hq_ + 2 * Hkv_) * D_, std=1.0)
            qn, kn = rnd(D_, std=1.0), rnd(D_, std=1.0)
            cos_t, sin_t = rnd(16384, D_, std=1.0), rnd(16384, D_, std=1.0)
            pos = torch.arange(T, dtype=torch.int64, device=dev)
            slots = torch.randperm(T, device=dev).to(torch.int32)
            kcache = rnd(T // page_, Hkv_, page_, D_).permute(0, 2, 1, 3)
            vcache = rnd(T // page_, Hkv_, page_, D_).permute(0, 2, 1, 3)
            qo = torch.empty(T, Hq_, D_, dtype=torch.bfloat16, device=dev)
            report(f"prefill q/k norm + rope + store T={T}",
                   timeit(lambda li: ops.qk_norm_rope_store(qkv, qn, kn, cos_t, sin_t, pos, slots, qo, kcache, vcache, Hq_, Hkv_, D_, 1e-6), n_layers=2),
                   T * (Hq_ + 2 * Hkv_) * D_ * 2 * 2 + T * D_ * 4)
        # causal attention over whole prompts: 8 sequences of 1024 tokens, paged cache
        Hq, Hkv, D, page, S, Lp = 32, 4, 128, 16, 8, 1024
        npg = S * Lp // page
        kc = rnd(npg, Hkv, page, D, std=1.0).permute(0, 2, 1, 3)
        vc = rnd(npg, Hkv, page, D, std=1.0).permute(0, 2, 1, 3)
        q = rnd(S * Lp, Hq, D, std=1.0)
        cu = torch.arange(0, S * Lp + 1, Lp, dtype=torch.int32, device=dev)
        used = torch.full((S,), Lp, dtype=torch.int32, device=dev)
        bt = torch.arange(npg, dtype=torch.int32, device=dev).view(S, Lp // page)
        out = torch.empty(S * Lp, Hq, D, dtype=torch.bfloat16, device=dev)
        report(f"prefill attention {S} x {Lp} tokens",
               timeit(lambda li: ops.paged_attention(q, kc, vc, cu, used, bt, D**-0.5, Lp, out=out), n_layers=2),
               flops=4 * S * Hq * D * Lp * (Lp + 1) // 2)
    if "mfma" in what:
        # the q/k/v projection of an 8192-token prefill chunk at the model's own shape
        M, N, K = 8192, 5120, 2048
        w_, xx = rnd(N, K), rnd(M, K, std=1.0)
        c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        report(f"prefill gemm qkv M={M} N={N} K={K}", timeit(lambda li: ops.gemm_nt(xx, w_, out=c), n_layers=2), flops=2 * M * N * K)
        del w_, xx, c
    if "prefill" in what or "configs" in what:
        # C3, chunked prefill: 16 sequences, a 512-token chunk on a cached prefix of 0..8192 tokens, Hq=32, Hkv=8
        Hq, Hkv, D, page, S, C = 32, 8, 128, 16, 16, 512
        rng = np.random.default_rng(3)
        prefix = rng.integers(0, 8193, size=S)
        Ls = prefix + C
        pages = [(int(n) + page - 1) // page for n in Ls]
        pool = sum(pages)
        perm = rng.permutation(pool)
        bt = np.full((S, max(pages)), -1, np.int32)
        o = 0
        for i, pg in enumerate(pages):
            bt[i, :pg] = perm[o : o + pg]
            o += pg
        kc = rnd(pool, Hkv, page, D, std=1.0).permute(0, 2, 1, 3)
        vc = rnd(pool, Hkv, page, D, std=1.0).permute(0, 2, 1, 3)
        q = rnd(S * C, Hq, D, std=1.0)
        cu = torch.arange(0, S * C + 1, C, dtype=torch.int32, device=dev)
        used = torch.tensor(Ls, dtype=torch.int32, device=dev)
        btd = torch.tensor(bt, device=dev)
        out = torch.empty(S * C, Hq, D, dtype=torch.bfloat16, device=dev)
        fl = 4 * Hq * D * int(sum(C * int(pf) + C * (C + 1) // 2 for pf in prefix))
        report(f"C3 chunked prefill attention 16 x 512 on prefixes (sum L={int(Ls.sum())})",
               timeit(lambda li: ops.paged_attention(q, kc, vc, cu, used, btd, D**-0.5, C, out=out), n_layers=2), flops=fl)
    if "small" in what:
        one = torch.zeros(64, dtype=torch.int32, device=dev)
        lib = _lib.load()
        report("one-element fill (node floor)",
               timeit(lambda li: _lib.check(lib.vx_fill_i32(one.data_ptr(), 1, 1, torch.cuda.current_stream().cuda_stream), "fill")), 4)
        x = rnd(B, H, std=1.0)
        res = rnd(B, H, std=1.0)
        wn = rnd(H, std=1.0)
        y = torch.empty_like(x)
        report("rms_norm", timeit(lambda li: ops.rms_norm(x, wn, 1e-6, hf_two_rounding=True, out=y)), 2 * B * H * 2)
        report("rms_norm + residual", timeit(lambda li: ops.rms_norm(x, wn, 1e-6, hf_two_rounding=True, residual=res, sum_out=res, out=y)),
               4 * B * H * 2)
        Hq, Hkv, D = 32, 4, 128
        qkv = rnd(B, (Hq + 2 * Hkv) * D, std=1.0)
        cos = rnd(4096, D, std=1.0)
        sin = rnd(4096, D, std=1.0)
        pos = torch.arange(B, device=dev)
        slot = torch.arange(B, device=dev, dtype=torch.int32)
        qo = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=dev)
        kcache = rnd(64, 16, Hkv, D)
        vcache = rnd(64, 16, Hkv, D)
        report("q/k norm + rope + cache store",
               timeit(lambda li: ops.qk_norm_rope_store(qkv, wn[:D], wn[:D], cos, sin, pos, slot, qo, kcache, vcache, Hq, Hkv, D, 1e-6)),
               2 * B * 5120 * 2)
        logits = rnd(B, 151936, std=1.0)
        report("greedy token + logprob", timeit(lambda li: ops.logprobs(logits, None, return_tokens=True)), B * 151936 * 2)
    if "configs" in what:
        # ---- the reference's other benchmark configurations, at their own shapes
        # C1: RMSNorm -> lm_head GEMM -> fp32 log_softmax on M rows (Qwen3-1.7B op chain)
        V = 151936
        wl = rnd(V, H)
        wn = rnd(H, std=1.0)
        for M in (1, 7, 64):
            x = rnd(M, H, std=1.0)
            hn = torch.empty_like(x)
            lg = torch.empty(M, V, dtype=torch.bfloat16, device=dev)
            report(f"C1 lm_head gemm M={M}", timeit(lambda li: ops.gemm_nt(x, wl, out=lg), n_layers=2), 2 * (V * H + M * H + M * V))
            lf = lg.float()
            report(f"C1 log_softmax fp32 M={M}", timeit(lambda li: ops.log_softmax(lf), n_layers=2), 2 * M * V * 4)
            report(f"C1 rms_norm M={M}", timeit(lambda li: ops.rms_norm(x, wn, 1e-6, hf_two_rounding=True, out=hn), n_layers=2),
                   2 * M * H * 2 + 2 * H)

            def chain(li):
                ops.rms_norm(x, wn, 1e-6, hf_two_rounding=True, out=hn)
                ops.gemm_nt(hn, wl, out=lg)
                ops.log_softmax(lg.float())

            report(f"C1 chain norm -> lm_head -> fp32 log_softmax M={M}", timeit(chain, n_layers=2),
                   2 * (V * H + M * H + M * V) + 2 * M * V * 4 + 2 * M * H * 2 + 2 * H)
        del wl
        # C2: decode attention, 64 sequences, context 128..4096, Hq=16, Hkv=8, D=128, page 16
        Hq, Hkv, D, page, S = 16, 8, 128, 16, 64
        rng = np.random.default_rng(2)
        L = rng.integers(128, 4097, size=S)
        pages = [(int(n) + page - 1) // page for n in L]
        pool = 32768
        perm = rng.permutation(pool)
        bt = np.full((S, 256), -1, np.int32)
        o = 0
        for i, pg in enumerate(pages):
            bt[i, :pg] = perm[o : o + pg]
            o += pg
        kc = rnd(pool, Hkv, page, D, std=1.0).permute(0, 2, 1, 3)
        vc = rnd(pool, Hkv, page, D, std=1.0).permute(0, 2, 1, 3)
        q = rnd(S, Hq, D, std=1.0)
        cu = torch.arange(S + 1, dtype=torch.int32, device=dev)
        used = torch.tensor(L, dtype=torch.int32, device=dev)
        btd = torch.tensor(bt, device=dev)
        out = torch.empty(S, Hq, D, dtype=torch.bfloat16, device=dev)
        order = torch.tensor(np.argsort(-L, kind="stable").astype(np.int32), device=dev)  # what the host metadata builder emits
        report(f"C2 decode attention B=64 (sum L={int(L.sum())})",
               timeit(lambda li: ops.paged_attention(q, kc, vc, cu, used, btd, D**-0.5, 1, out=out, seq_order=order), n_layers=2),
               int(L.sum()) * 2 * Hkv * D * 2 + 2 * S * Hq * D * 2 + sum(pages) * 4)
        del kc, vc
        # C4: fused MoE block at T tokens
        gu = rnd(E, 2 * I, H + 64)[..., :H]
        dn = rnd(E, H, I)
        for T in (1, 64, 256, 4096):
            x = rnd(T, H, std=1.0)
            logits = torch.randn(T, E, generator=g, device=dev)
            w, idx = ops.router_topk(logits, k, index_dtype=torch.int32)
            U = int(torch.unique(idx).numel())
            y = torch.empty_like(x)
            t = timeit(lambda li: ops.fused_moe(x, w, idx, gu[:, :I, :], gu[:, I:, :], dn, E, out=y), n_layers=2)
            report(f"C4 fused MoE T={T} ({U} experts)", t, U * 3 * H * I * 2 + 2 * T * H * 2 + T * k * 6)
            if T == 4096 and t is not None:
                report(f"C4 fused MoE T={T}, as flops", t, flops=T * k * 6 * H * I)
    if "other" in what:
        # fp32 / fp16 matrix-core GEMM (one 64 x 64 x 32 tile shape for every M)
        for dt, nm in ((torch.float32, "fp32"), (torch.float16, "fp16")):
            for M in (256, 4096):
                xx = torch.randn(M, 4096, generator=g, device=dev).to(dt)
                ww = (torch.randn(4096, 4096, generator=g, device=dev) * 0.02).to(dt)
                report(f"{nm} gemm M={M} N=4096 K=4096", timeit(lambda li: ops.matmul(xx, ww.t()), n_layers=2), flops=2 * M * 4096 * 4096)
    if "dropin" in what:
        results.extend(dropin_decode(a, quiet, layouts=(True,) if a.dropin_head_major else None))
    if "trainlayer" in what:
        results.extend(dropin_train_layers(quiet))
    if "copy" in what:
        # a plain device copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        report("copy 1 GiB", timeit(lambda li: dst.copy_(src), n_layers=2), 2 << 30)
    return results


def dropin_decode(a, quiet: bool = False, layouts=None) -> list:
    """What a caller of the reference gets by switching imports: a HuggingFace ``Qwen3MoeForCausalLM`` of the
    30B-A3B shape (random weights, built on the GPU) behind the registered attention function, the patched MoE
    block and batch-invariant mode, one decode step of ``--batch`` sequences (contexts U[256, 2048], page 16)
    captured in a HIP graph - once with ``max_seqlen_q = 1`` and once the way the reference's CudaGraphManager
    captures it (``max_seqlen_q`` = the bucket's tokens, vexact/inferencer/cudagraph_utils.py:163)."""
    import types

    import numpy as np
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS
    from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeForCausalLM

    from vexact_amd.batch_invariant_ops import flash_attention_forward, set_batch_invariant_mode
    from vexact_amd.batch_invariant_ops.kv_cache_context import KVCacheStore, clear_kv_cache_context, set_kv_cache_context
    from vexact_amd.models.qwen3_moe import apply_qwen3_moe_patches, fuse_qkv_weights, remove_qwen3_moe_patches

    say = (lambda *x, **k: None) if quiet else print
    B, page = a.batch, a.page
    cfg = Qwen3MoeConfig(vocab_size=151936, hidden_size=2048, intermediate_size=6144, num_hidden_layers=48,
                         num_attention_heads=32, num_key_value_heads=4, head_dim=128, num_experts=128, num_experts_per_tok=8,
                         moe_intermediate_size=768, norm_topk_prob=True, max_position_embeddings=40960, rms_norm_eps=1e-6,
                         rope_parameters={"rope_type": "default", "rope_theta": 1.0e6})
    cfg._attn_implementation = "triton-invariant"
    ALL_ATTENTION_FUNCTIONS["triton-invariant"] = flash_attention_forward
    apply_qwen3_moe_patches()
    with torch.device("meta"):
        model = Qwen3MoeForCausalLM(cfg)
    model = model.to_empty(device="cuda").eval()
    g = torch.Generator(device="cuda").manual_seed(5)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if "norm" in name:
                p.fill_(1.0)
            else:
                p.normal_(0.0, 0.02, generator=g)
    for p in model.parameters():
        p.data = p.data.to(torch.bfloat16)
    rot = model.model.rotary_emb  # inv_freq is a non-persistent buffer, which to_empty() leaves uninitialised
    inv = 1.0 / (1.0e6 ** (torch.arange(0, 128, 2, device="cuda").float() / 128))
    rot.inv_freq, rot.original_inv_freq = inv, inv.clone()
    for layer in model.model.layers:
        layer.mlp.experts.pack_for_decode()
    fuse_qkv_weights(model)  # the optional load-time step: one q/k/v projection per layer instead of three
    rng = np.random.default_rng(5)
    lens = rng.integers(256, 2049, size=B)
    pages = [(int(n) + 2 + page - 1) // page for n in lens]
    pool = sum(pages) + 8
    perm, bt, o = rng.permutation(pool), np.zeros((B, max(pages)), np.int32), 0
    for i, pg in enumerate(pages):
        bt[i, :pg] = perm[o:o + pg]
        o += pg
    i32 = dict(dtype=torch.int32, device="cuda")
    ids = torch.randint(0, cfg.vocab_size, (1, B), device="cuda")
    pos = torch.as_tensor(lens, device="cuda").long()[None]
    bt_d, ctx = torch.as_tensor(bt).cuda(), torch.as_tensor(lens + 1, **i32)
    slot = torch.as_tensor([bt[i, lens[i] // page] * page + lens[i] % page for i in range(B)], **i32)
    qsl = torch.arange(B + 1, **i32)

    def forward():
        out = model.model(input_ids=ids, position_ids=pos, use_cache=False, return_dict=True)
        return model.lm_head(out.last_hidden_state)

    res = []
    layouts = (False, True) if layouts is None else layouts
    for head_major in layouts:
        store = KVCacheStore(cfg, types.SimpleNamespace(page_size=page, max_cache_blocks=pool), torch.device("cuda"),
                             head_major=head_major)
        for t in list(store.key_cache.values()) + list(store.value_cache.values()):
            t.normal_(0, 1)
        where = "KVCacheStore(head_major=True)" if head_major else "the reference's cache layout"
        # the reference's CudaGraphManager captures with max_seqlen_q = the bucket's tokens (cudagraph_utils.py:163)
        for msq, how in ((1, "max_seqlen_q = 1"), (B, "max_seqlen_q = bucket tokens"))[: 1 if head_major else 2]:
            set_kv_cache_context(is_paged_attn=True, key_cache=store.key_cache, value_cache=store.value_cache, block_tables=bt_d,
                                 context_lens=ctx, slot_mapping=slot, query_start_loc=qsl, max_seqlen_q=msq)
            try:
                with torch.inference_mode(), set_batch_invariant_mode(True):
                    forward()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        forward()
                    for _ in range(3):
                        graph.replay()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(10):
                        graph.replay()
                    e1.record()
                    torch.cuda.synchronize()
            finally:
                clear_kv_cache_context()
            ms = e0.elapsed_time(e1) / 10
            say(f"HF Qwen3MoeForCausalLM drop-in decode, batch {B}, {where}, {how}: {ms:.2f} ms/step = {B / ms * 1e3:.0f} tok/s", flush=True)
            res.append({"name": f"HF drop-in decode step, batch {B}, {where}, {how}", "us": round(ms * 1e3, 1),
                        "ms_per_step": round(ms, 3), "tok_s": round(B / ms * 1e3), "head_major": head_major, "max_seqlen_q": msq})
            del graph
        del store
        torch.cuda.empty_cache()
    del model
    torch.cuda.empty_cache()
    remove_qwen3_moe_patches()
    return res


def dropin_train_layers(quiet: bool = False, layers: int = 2, seqs: int = 8, seq_len: int = 1024) -> list:
    """The trainer's side of the drop-in: ``layers`` HuggingFace ``Qwen3MoeDecoderLayer``s of the 30B-A3B shape under
    the patches, batch-invariant mode and a packed (cache-less) context, forward + backward over ``seqs`` sequences of
    ``seq_len`` tokens; and the paged prefill of the same tokens in inference mode for comparison."""
    import types

    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS
    from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeForCausalLM

    from vexact_amd.batch_invariant_ops import flash_attention_forward, set_batch_invariant_mode
    from vexact_amd.batch_invariant_ops.kv_cache_context import KVCacheStore, clear_kv_cache_context, set_kv_cache_context
    from vexact_amd.models.qwen3_moe import apply_qwen3_moe_patches

    say = (lambda *x, **k: None) if quiet else print
    cfg = Qwen3MoeConfig(vocab_size=32000, hidden_size=2048, intermediate_size=6144, num_hidden_layers=layers,
                         num_attention_heads=32, num_key_value_heads=4, head_dim=128, num_experts=128, num_experts_per_tok=8,
                         moe_intermediate_size=768, norm_topk_prob=True, max_position_embeddings=40960, rms_norm_eps=1e-6,
                         rope_parameters={"rope_type": "default", "rope_theta": 1.0e6})
    cfg._attn_implementation = "triton-invariant"
    ALL_ATTENTION_FUNCTIONS["triton-invariant"] = flash_attention_forward
    apply_qwen3_moe_patches()
    with torch.device("meta"):
        model = Qwen3MoeForCausalLM(cfg)
    model = model.to_empty(device="cuda")
    g = torch.Generator(device="cuda").manual_seed(5)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if "norm" in name:
                p.fill_(1.0)
            else:
                p.normal_(0.0, 0.02, generator=g)
    for p in model.parameters():
        p.data = p.data.to(torch.bfloat16)
    rot = model.model.rotary_emb
    inv = 1.0 / (1.0e6 ** (torch.arange(0, 128, 2, device="cuda").float() / 128))
    rot.inv_freq, rot.original_inv_freq = inv, inv.clone()
    T, page = seqs * seq_len, 16
    i32 = dict(dtype=torch.int32, device="cuda")
    ctx, qsl = torch.full((seqs,), seq_len, **i32), torch.arange(0, T + 1, seq_len, **i32)
    pos = torch.arange(seq_len, device="cuda").repeat(seqs)[None]
    x0 = torch.randn(1, T, 2048, device="cuda", generator=g).to(torch.bfloat16)
    dy = torch.randn(1, T, 2048, device="cuda", generator=g).to(torch.bfloat16)

    def through_layers(x):
        pe = rot(x, pos)
        for layer in model.model.layers:
            x = layer(x, position_ids=pos, position_embeddings=pe)
        return x

    def train_step():
        for p in model.parameters():
            p.grad = None
        through_layers(x0.clone().requires_grad_()).backward(dy)

    def timed(fn, reps=5):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    res = []
    set_kv_cache_context(is_paged_attn=False, context_lens=ctx, query_start_loc=qsl, max_seqlen_q=seq_len)
    try:
        with set_batch_invariant_mode(True):
            ms = timed(train_step)
    finally:
        clear_kv_cache_context()
    say(f"HF decoder layer, trainer forward + backward, {seqs} x {seq_len} packed tokens: {ms / layers:.2f} ms per layer", flush=True)
    res.append({"name": f"HF decoder layer forward + backward, {seqs} x {seq_len} tokens", "us": round(ms / layers * 1e3, 1)})
    pages = seq_len // page
    store = KVCacheStore(cfg, types.SimpleNamespace(page_size=page, max_cache_blocks=seqs * pages + 4), torch.device("cuda"))
    set_kv_cache_context(is_paged_attn=True, key_cache=store.key_cache, value_cache=store.value_cache,
                         block_tables=torch.arange(seqs * pages, **i32).reshape(seqs, pages), context_lens=ctx,
                         slot_mapping=torch.arange(T, **i32), query_start_loc=qsl, max_seqlen_q=seq_len)
    try:
        with torch.inference_mode(), set_batch_invariant_mode(True):
            ms = timed(lambda: through_layers(x0))
    finally:
        clear_kv_cache_context()
    say(f"HF decoder layer, paged prefill of the same tokens (inference mode): {ms / layers:.2f} ms per layer", flush=True)
    res.append({"name": f"HF decoder layer paged prefill, {seqs} x {seq_len} tokens", "us": round(ms / layers * 1e3, 1)})
    return res


def main() -> None:
    run(parse())


if __name__ == "__main__":
    main()
