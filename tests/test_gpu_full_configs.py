"""GPU parity at the full sizes of the benchmark configurations.

The oracle cannot run these shapes whole in seconds, so each test checks (a) the size-independent
properties at full size - a sequence alone vs in the batch, the last row of a prefill chunk vs the decode
step of the same token, the first T rows of a smaller token count vs the same rows of the large one: 0
differing bits - and (b) a subsample of rows against the CPU oracle (attention: atol = rtol = 3e-3, the
reference's own bound against eager attention; MoE: 2 bf16 ulp; integer outputs exact). Inputs are drawn
once (seeded) and both sides see the same bits.
"""

import pytest
import torch

from oracle import attention as OA
from oracle import moe as OM
from oracle import row_ops as OR
from tests.util import assert_bf16_close, assert_bitwise, ulp_histogram

pytestmark = pytest.mark.gpu

from vexact_amd import ops  # noqa: E402
from vexact_amd.batch_invariant_ops import triton_flash_attn_varlen_func as flash_attn_varlen_func  # noqa: E402
from vexact_amd.batch_invariant_ops.fused_moe import fused_moe_forward  # noqa: E402


def _cu(lens):
    return torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)


def _exact_attention_rows(q_rows, k_seq, v_seq, scale):
    """Causal attention of the LAST len(q_rows) positions of a sequence in float64 with no rounding anywhere: the
    exact result that both the kernel and the eager oracle approximate. ``q_rows [Q, Hq, D]``, ``k_seq / v_seq [K, Hkv, D]``."""
    q, k, v = q_rows.double().transpose(0, 1), k_seq.double().transpose(0, 1), v_seq.double().transpose(0, 1)
    g = q.shape[0] // k.shape[0]
    k, v = k.repeat_interleave(g, dim=0), v.repeat_interleave(g, dim=0)
    s = torch.matmul(q, k.transpose(-1, -2)) * scale
    ql, kl = q.shape[1], k.shape[1]
    mask = torch.arange(kl)[None, :] <= (torch.arange(ql) + (kl - ql))[:, None]
    s = s.masked_fill(~mask[None], float("-inf"))
    return torch.matmul(torch.softmax(s, -1), v).transpose(0, 1)


def _assert_no_worse_than_eager(got, eager, exact, what):
    """Both the kernel (like the reference's kernel: un-normalised probabilities rounded to bf16, normalised at the end)
    and the eager oracle (normalised probabilities rounded) approximate the exact result. Many elements lie more than
    2 bf16 ulps from the eager oracle because outputs over thousands of keys are averages near 0 and the two round in
    different places. This shows that the kernel's distance from the exact result is of the size of the eager
    oracle's own: per (row, head), max |kernel - exact| <= 1.5 max |eager - exact| + 2^-9 max |exact|."""
    ek = (got.double() - exact).abs().amax(-1)
    ee = (eager.double() - exact).abs().amax(-1)
    bound = 1.5 * ee + 2.0 ** -9 * exact.abs().amax(-1)
    print(f"[exact] {what}: max |kernel - exact| {float(ek.max()):.3e} (mean {float(ek.mean()):.3e}), "
          f"max |eager - exact| {float(ee.max()):.3e} (mean {float(ee.mean()):.3e}) over {ek.numel()} (row, head) pairs", flush=True)
    bad = ek > bound
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} (row, head) pairs beyond the bound; worst {float((ek - bound).max()):.3e}"


def _bf16_normal(shape, seed):
    """Drawn on the GPU (the CPU generator would take minutes at these sizes); the CPU copy has the same bits."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    t = torch.empty(shape, dtype=torch.bfloat16, device="cuda")
    t.normal_(0.0, 1.0, generator=g)
    return t


def test_config1_op_chain_full_size():
    # Qwen3-1.7B op chain at hidden 2048, vocabulary 151936: RMSNorm -> lm_head -> .float() -> log_softmax on the
    # first M rows of ONE 64-row draw, M = 1 / 7 / 64; both RMSNorm forms: HuggingFace's module arithmetic under the
    # aten overrides (its mean goes through mean_dim, two roundings) and batch_invariant_rms_norm (one rounding)
    from vexact_amd.batch_invariant_ops import batch_invariant_rms_norm, set_batch_invariant_mode

    H, V = 2048, 151936
    g = torch.Generator().manual_seed(1)
    x = torch.randn(64, H, generator=g).to(torch.bfloat16)
    wn = (1 + 0.02 * torch.randn(H, generator=g)).to(torch.bfloat16)
    W_t = _bf16_normal((V, H), 11) * 0.02  # contiguous [V, H]; the chain multiplies by W_t.t()
    xd, wnd = x.cuda(), wn.cuda()

    def hf_norm(t):  # the module's forward, op by op
        t32 = t.to(torch.float32)
        var = t32.pow(2).mean(-1, keepdim=True)
        return wnd * (t32 * torch.rsqrt(var + 1e-6)).to(t.dtype)

    def chain(t, form):
        h = hf_norm(t) if form == "hf" else batch_invariant_rms_norm(t, wnd, 1e-6)
        logits = torch.mm(h, W_t.t())
        return h, logits, torch.log_softmax(logits.float(), dim=-1)

    W_cpu = W_t.cpu()
    for form in ("hf", "one-rounding"):
        with set_batch_invariant_mode(True):
            outs = {M: chain(xd[:M], form) for M in (1, 7, 64)}
        full = outs[64]
        for M in (1, 7):
            for name, a, b in zip(("norm", "logits", "log_softmax"), outs[M], full):
                assert_bitwise(a, b[:M], f"{form}: {name} rows at M={M} vs the same rows at M=64")
        # against the CPU oracle on the same bits
        h_ref = OR.hf_rms_norm_ref(x, wn) if form == "hf" else OR.rms_norm_ref(x, wn)
        ulp_histogram(full[0], h_ref, f"C1 {form} RMSNorm vs oracle")
        assert_bf16_close(full[0], h_ref, max_ulp=1, atol_frac=0.0, what=f"{form} RMSNorm")
        logits_ref = OR.matmul_ref(full[0].cpu(), W_cpu.t())  # the GEMM on the kernel's own normalised rows
        hist = ulp_histogram(full[1], logits_ref, f"C1 {form} logits [64, 151936] vs oracle")
        # <= 2 bf16 ulp; the few elements beyond sit where the 2048-term sum cancels to a small number
        assert hist[">2"] <= 1e-4
        assert_bf16_close(full[1], logits_ref, max_ulp=2, atol_frac=1e-3, what=f"{form} logits")
        lp_ref = OR.log_softmax_ref(full[1].cpu().float())
        assert float((full[2].cpu() - lp_ref).abs().max()) <= 2e-5, "log_softmax of the kernel's logits vs oracle"
        lp_chain = OR.log_softmax_ref(OR.matmul_ref(h_ref, W_cpu.t()).float())
        assert float((full[2].cpu() - lp_chain).abs().max()) <= 2e-2, "whole chain logprob vs oracle"


def test_config5_full_model_batch_256_equals_batch_1():
    # the whole 48-layer Qwen3-30B-A3B-shaped decoder: one graph-captured decode step at batch 256 against every
    # request alone at batch 1 (eager): 0 differing logprob bits, same greedy token
    import bench

    wl = bench.build_workload(layers=48, batch=256, seed=5, log=False)
    db = wl.dec.bucket(wl.B, wl.B)
    db.load(wl.dmeta, wl.first_tokens)
    graph = wl.dec.capture(db, 1)
    for rep in range(2):
        db.logprobs.zero_()
        graph.replay()
        torch.cuda.synchronize()
        lp, tok = db.logprobs.cpu().clone(), db.tokens.cpu().clone()
        if rep == 0:
            lp0, tok0 = lp, tok
        else:
            assert_bitwise(lp, lp0, "second replay of the decode graph")
    assert bool(torch.isfinite(lp0).all()) and bool((lp0 < 0).all())
    bits, checked = bench.drift_check(wl, lp0, tok0, 256)
    assert checked == 256 and bits == 0, f"{bits} differing bits over {checked} requests"
    del wl, db, graph
    torch.cuda.empty_cache()


def test_config2_paged_decode_full_size():
    # 16 query / 8 kv heads, head size 128, page 16, 64 sequences of 128..4096 keys, block tables =
    # consecutive slices of a random permutation of a 32768-page pool
    g = torch.Generator().manual_seed(2)
    B, Hq, Hkv, D, page, pool = 64, 16, 8, 128, 16, 32768
    kv_lens = torch.randint(128, 4097, (B,), generator=g)
    pages = (kv_lens + page - 1) // page
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    table = torch.full((B, 256), -1, dtype=torch.int32)
    o = 0
    for s in range(B):
        table[s, : int(pages[s])] = perm[o : o + int(pages[s])]
        o += int(pages[s])
    k_cache, v_cache = _bf16_normal((pool, page, Hkv, D), 21), _bf16_normal((pool, page, Hkv, D), 22)
    q = _bf16_normal((B, Hq, D), 23)
    used = kv_lens.to(torch.int32)
    cu = _cu([1] * B)
    out, _ = flash_attn_varlen_func(q, k_cache, v_cache, cu_seqlens_q=cu.cuda(), max_seqlen_q=1, seqused_k=used.cuda(),
                                    page_table=table.cuda(), causal=True)
    one_cu = _cu([1]).cuda()
    for s in range(B):
        one, _ = flash_attn_varlen_func(q[s : s + 1], k_cache, v_cache, cu_seqlens_q=one_cu, max_seqlen_q=1,
                                        seqused_k=used[s : s + 1].cuda(), page_table=table[s : s + 1].cuda(), causal=True)
        assert_bitwise(one[0], out[s], f"sequence {s} alone vs in the batch of 64")
    sub = [0, 17, 40, 63]
    kc, vc = k_cache.cpu(), v_cache.cpu()
    ref = OA.paged_attention_ref(q[sub].cpu(), kc, vc, _cu([1] * len(sub)), used[sub], table[sub], D**-0.5)
    # tolerance of the reference's own paged-vs-eager test (test_triton_attention_varlen.py:390-415): the eager
    # oracle rounds normalised probabilities, the kernel un-normalised ones, over up to 4096 keys
    torch.testing.assert_close(out[sub].cpu().float(), ref.float(), atol=3e-3, rtol=3e-3)
    ulp_histogram(out[sub], ref, "C2 decode attention rows vs eager oracle")
    # what the many elements beyond 2 ulp are: both sides measured against the exact (float64) result
    exact = torch.cat([_exact_attention_rows(q[s : s + 1].cpu(), OA.gather_paged(kc, table[s], int(used[s])),
                                             OA.gather_paged(vc, table[s], int(used[s])), D**-0.5) for s in sub])
    _assert_no_worse_than_eager(out[sub].cpu(), ref, exact, "C2 decode attention rows")


def test_config3_chunked_prefill_full_size():
    # 32 query / 8 kv heads, head size 128, 16 sequences, a 512-token chunk appended to prefixes of 0..8192 keys
    g = torch.Generator().manual_seed(3)
    S, Hq, Hkv, D, page, C = 16, 32, 8, 128, 16, 512
    prefix = torch.randint(0, 8193, (S,), generator=g)
    prefix[0], prefix[1] = 0, 8192  # both ends of the range
    kv_lens = (prefix + C).tolist()
    pages = [(n + page - 1) // page for n in kv_lens]
    total = sum(pages) + 100
    perm = torch.randperm(total, generator=g).to(torch.int32)
    table = torch.full((S, max(pages)), -1, dtype=torch.int32)
    o = 0
    for s in range(S):
        table[s, : pages[s]] = perm[o : o + pages[s]]
        o += pages[s]
    k_cache, v_cache = _bf16_normal((total, page, Hkv, D), 31), _bf16_normal((total, page, Hkv, D), 32)
    q = _bf16_normal((S * C, Hq, D), 33)
    used = torch.tensor(kv_lens, dtype=torch.int32)
    cu = _cu([C] * S)
    out, _ = flash_attn_varlen_func(q, k_cache, v_cache, cu_seqlens_q=cu.cuda(), max_seqlen_q=C, seqused_k=used.cuda(),
                                    page_table=table.cuda(), causal=True)
    # a sequence alone on the same pages
    for s in (0, 1, 7):
        one, _ = flash_attn_varlen_func(q[s * C : (s + 1) * C], k_cache, v_cache, cu_seqlens_q=_cu([C]).cuda(), max_seqlen_q=C,
                                        seqused_k=used[s : s + 1].cuda(), page_table=table[s : s + 1].cuda(), causal=True)
        assert_bitwise(one, out[s * C : (s + 1) * C], f"chunk of sequence {s} alone vs in the batch")
    # the last row of every chunk is the decode step of that token
    last = torch.arange(S) * C + C - 1
    dec, _ = flash_attn_varlen_func(q[last.cuda()], k_cache, v_cache, cu_seqlens_q=_cu([1] * S).cuda(), max_seqlen_q=1,
                                    seqused_k=used.cuda(), page_table=table.cuda(), causal=True)
    assert_bitwise(dec, out[last.cuda()], "last row of each chunk vs decode")
    # oracle on a few rows: row i of a chunk is the last row of attention over the first prefix + i + 1 keys
    kc, vc, qc = k_cache.cpu(), v_cache.cpu(), q.cpu()
    got_rows, ref_rows, exact_rows = [], [], []
    for s in (0, 1, 5):
        ks = OA.gather_paged(kc, table[s], kv_lens[s])
        vs = OA.gather_paged(vc, table[s], kv_lens[s])
        for i in (0, 255, C - 1):
            n = int(prefix[s]) + i + 1
            ref = OA.eager_attention(qc[s * C + i : s * C + i + 1], ks[:n], vs[:n], D**-0.5)
            torch.testing.assert_close(out[s * C + i : s * C + i + 1].cpu().float(), ref.float(), atol=3e-3, rtol=3e-3,
                                       msg=lambda m: f"sequence {s} chunk row {i} vs eager oracle: {m}")
            got_rows.append(out[s * C + i : s * C + i + 1].cpu())
            ref_rows.append(ref)
            exact_rows.append(_exact_attention_rows(qc[s * C + i : s * C + i + 1], ks[:n], vs[:n], D**-0.5))
    ulp_histogram(torch.cat(got_rows), torch.cat(ref_rows), "C3 chunked prefill rows vs eager oracle")
    _assert_no_worse_than_eager(torch.cat(got_rows), torch.cat(ref_rows), torch.cat(exact_rows), "C3 chunked prefill rows")


def test_config4_fused_moe_full_size():
    # hidden 2048, 128 experts, top-8, intermediate 768; token counts 1 / 64 / 256 / 4096 = first rows of one draw
    T, H, I, E, k = 4096, 2048, 768, 128, 8
    x = _bf16_normal((T, H), 41)
    g = torch.Generator().manual_seed(4)
    logits = torch.randn(T, E, generator=g)
    gate_up = _bf16_normal((E, 2 * I, H), 42) * 0.02
    down = _bf16_normal((E, H, I), 43) * 0.02
    w_ref, i_ref = OM.router_ref(logits, k)
    w, idx = ops.router_topk(logits.cuda(), k, renorm=True, index_dtype=torch.int64)
    # rows where the oracle's fp32 probabilities collide for distinct logits are excluded (as in the router test)
    p = torch.softmax(logits, -1)
    srt = torch.sort(p, dim=-1, descending=True, stable=True).values
    lsrt = torch.sort(logits, dim=-1, descending=True, stable=True).values
    clean = ~(((srt[:, 1 : k + 1] == srt[:, :k]) & (lsrt[:, 1 : k + 1] != lsrt[:, :k])).any(-1))
    assert clean.float().mean() > 0.99
    assert torch.equal(idx.cpu()[clean], i_ref[clean]), "top-8 indices"
    assert_bf16_close(w.cpu()[clean], w_ref[clean], max_ulp=1, what="routing weights")
    full = fused_moe_forward(E, w, idx, x, None, None, down, fc1_1_2_weight=gate_up)
    for t in (1, 64, 256):
        part = fused_moe_forward(E, w[:t], idx[:t], x[:t], None, None, down, fc1_1_2_weight=gate_up)
        assert_bitwise(part, full[:t], f"first {t} tokens vs the same rows at 4096")
    packed = (ops.pack_expert_weights(gate_up), ops.pack_expert_weights(down))
    for t in (1, 256):
        part = fused_moe_forward(E, w[:t], idx[:t], x[:t], None, None, down, fc1_1_2_weight=gate_up, packed_weights=packed)
        assert_bitwise(part, full[:t], f"first {t} tokens on packed expert weights")
    rows = torch.tensor([0, 63, 255, 1000, 4095])
    gu = gate_up.cpu()
    ref = OM.fused_moe_ref(x.cpu()[rows], w.cpu()[rows], idx.cpu()[rows], gu[:, :I], gu[:, I:], down.cpu())
    ulp_histogram(full[rows.cuda()], ref, "C4 fused MoE rows vs fused-order oracle")
    assert_bf16_close(full[rows.cuda()], ref, max_ulp=2, atol_frac=2e-3, what="config-4 rows vs fused-order oracle")
