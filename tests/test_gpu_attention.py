"""GPU parity: paged / packed attention and the KV-cache scatter.

Restates tests/batch_invariant_ops/test_triton_attention_varlen.py of the reference: paged vs
eager oracle (atol = rtol = 3e-3 at |x| ~ 0.1, :390-415) and alone vs in-batch bitwise (:417-421),
alias equality (:424-432), prefill last row == decode row bitwise (:435-454), the Qwen3-like
16q/8kv/128 page-256 case incl. the packed twin (:457-493), MLA 192/128 (:496-558), backward raises
(:561-569), wrapper shape (:572-598), error messages (:201-211, :24-30).
"""

import pytest
import torch

from oracle import attention as OA
from tests.util import assert_bf16_close, assert_bitwise

pytestmark = pytest.mark.gpu

from vexact_amd.batch_invariant_ops import flash_attention_forward, triton_flash_attn_varlen_func as flash_attn_varlen_func  # noqa: E402
from vexact_amd.batch_invariant_ops.kv_cache_context import (  # noqa: E402
    clear_kv_cache_context,
    set_kv_cache_context,
    store_kvcache,
)


def _cu(lens):
    out = [0]
    for n in lens:
        out.append(out[-1] + n)
    return torch.tensor(out, dtype=torch.int32)


def _run_paged(q_seqs, k_seqs, v_seqs, page_size, page_kw="page_table", perm=None, max_seqlen_q=None, pad_seqs=0):
    k_cache, v_cache, table = OA.make_paged_kv_cache(k_seqs, v_seqs, page_size, perm=perm)
    q_lens = [q.shape[0] for q in q_seqs]
    kv_lens = [k.shape[0] for k in k_seqs]
    cu = _cu(q_lens)
    used = torch.tensor(kv_lens, dtype=torch.int32)
    if pad_seqs:  # graph-style padding: zero-length rows pointing at page 0
        cu = torch.cat([cu, cu[-1:].repeat(pad_seqs)])
        used = torch.cat([used, torch.zeros(pad_seqs, dtype=torch.int32)])
        table = torch.cat([table, torch.zeros(pad_seqs, table.shape[1], dtype=torch.int32)])
    out, _ = flash_attn_varlen_func(
        torch.cat(q_seqs, dim=0).cuda(), k_cache.cuda(), v_cache.cuda(), cu_seqlens_q=cu.cuda(),
        max_seqlen_q=max(q_lens) if max_seqlen_q is None else max_seqlen_q, seqused_k=used.cuda(),
        causal=True, **{page_kw: table.cuda()},
    )
    return out


def _seqs(lens, heads, dim, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(n, heads, dim, generator=g) * scale).to(torch.bfloat16) for n in lens]


@pytest.mark.parametrize(
    ("q_lens", "kv_lens"),
    [([1, 1, 1, 1], [17, 31, 40, 49]), ([24, 19], [24, 19]), ([24, 1, 17, 1], [24, 33, 17, 41]),
     ([1, 1, 1], [255, 256, 257]), ([300, 5, 1], [300, 700, 1000])],
)
def test_paged_correctness_and_batch_invariance(q_lens, kv_lens):
    qh, kh, d, page = 4, 2, 32, 16
    q = _seqs(q_lens, qh, d, 1, 0.1)
    k = _seqs(kv_lens, kh, d, 2, 0.1)
    v = _seqs(kv_lens, kh, d, 3, 0.1)
    out = _run_paged(q, k, v, page)
    ref = torch.cat([OA.eager_attention(a, b, c, d**-0.5) for a, b, c in zip(q, k, v)], dim=0)
    torch.testing.assert_close(out.cpu(), ref, atol=3e-3, rtol=3e-3)
    off = 0
    for a, b, c in zip(q, k, v):
        one = _run_paged([a], [b], [c], page)
        assert_bitwise(out[off : off + a.shape[0]], one, "alone vs batch")
        off += a.shape[0]
    # the general kernel gives the decode kernel's bits (max_seqlen_q unknown -> general path)
    if max(q_lens) == 1:
        assert_bitwise(_run_paged(q, k, v, page, max_seqlen_q=0), out, "general kernel on decode batch")
    # padded sequences are no-ops
    assert_bitwise(_run_paged(q, k, v, page, pad_seqs=3), out, "padded sequence rows")


@pytest.mark.parametrize(("qh", "kh", "d"), [(4, 2, 32), (8, 2, 128), (32, 4, 128)])
def test_general_launch_over_prefill_chunks_and_decode_tokens(qh, kh, d):
    # what a scheduler with chunked prefill hands over: a few chunks of very different lengths among single decode
    # tokens. The launch numbers its (sequence, row block) pairs compactly and gives the single-token sequences to
    # the decode kernel; every sequence keeps the bits it has alone, in the general and in the decode launch.
    page = 16
    q_lens = [200, 1, 1, 33, 1, 64, 1, 1, 7, 1, 1, 130]
    prefix = [0, 700, 15, 100, 255, 1, 256, 31, 300, 1024, 0, 77]
    kv_lens = [a + b for a, b in zip(q_lens, prefix)]
    q = _seqs(q_lens, qh, d, 51, 0.1)
    k = _seqs(kv_lens, kh, d, 52, 0.1)
    v = _seqs(kv_lens, kh, d, 53, 0.1)
    out = _run_paged(q, k, v, page)
    ref = torch.cat([OA.eager_attention(a, b, c, d**-0.5) for a, b, c in zip(q, k, v)], dim=0)
    torch.testing.assert_close(out.cpu(), ref, atol=3e-3, rtol=3e-3)
    off = 0
    for a, b, c in zip(q, k, v):
        one = _run_paged([a], [b], [c], page)  # a single token alone runs as a decode launch
        assert_bitwise(out[off : off + a.shape[0]], one, "alone vs in the mixed batch")
        off += a.shape[0]
    assert_bitwise(_run_paged(q, k, v, page, pad_seqs=5), out, "padded sequence rows")
    assert_bitwise(_run_paged(q, k, v, page, max_seqlen_q=sum(q_lens)), out, "max_seqlen_q = the batch's tokens")
    # a decode batch launched the general way (max_seqlen_q = the bucket's tokens, as a captured graph has it)
    qd = [t[-1:] for t in q]
    dec = _run_paged(qd, k, v, page)
    assert_bitwise(_run_paged(qd, k, v, page, max_seqlen_q=64, pad_seqs=4), dec, "decode batch through a general launch")
    off = 0
    for i, a in enumerate(q):
        assert_bitwise(dec[i : i + 1], out[off + a.shape[0] - 1 : off + a.shape[0]], "last chunk row vs decode step")
        off += a.shape[0]
    # a sequence order (longest context first) for the decode kernel inside the general launch changes nothing
    from vexact_amd import ops
    k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, page)
    order = torch.argsort(torch.tensor(kv_lens), descending=True, stable=True).to(torch.int32).cuda()
    ordered = ops.paged_attention(torch.cat(q, dim=0).cuda(), k_cache.cuda(), v_cache.cuda(), _cu(q_lens).cuda(),
                                  torch.tensor(kv_lens, dtype=torch.int32).cuda(), table.cuda(), d**-0.5, max(q_lens),
                                  seq_order=order)
    assert_bitwise(ordered, out, "general launch with a sequence order")


def test_page_table_aliases_match():
    q, k, v = _seqs([1], 4, 32, 4), _seqs([33], 2, 32, 5), _seqs([33], 2, 32, 6)
    assert_bitwise(_run_paged(q, k, v, 16, page_kw="page_table"), _run_paged(q, k, v, 16, page_kw="block_table"), "alias")


@pytest.mark.parametrize("qh,kh,d,page,kv_lens", [(4, 2, 32, 16, [17, 33, 64]), (16, 8, 128, 256, list(range(74, 83))),
                                                    (32, 4, 128, 16, [250, 256, 257, 600, 1030])])
def test_prefill_decode_and_packed_bitwise_alignment(qh, kh, d, page, kv_lens):
    qp = _seqs(kv_lens, qh, d, 7)
    k = _seqs(kv_lens, kh, d, 8)
    v = _seqs(kv_lens, kh, d, 9)
    prefill = _run_paged(qp, k, v, page)
    decode = _run_paged([x[-1:] for x in qp], k, v, page)
    cu = _cu(kv_lens).cuda()
    packed, _ = flash_attn_varlen_func(
        torch.cat(qp).cuda(), torch.cat(k).cuda(), torch.cat(v).cuda(), cu_seqlens_q=cu, cu_seqlens_k=cu,
        max_seqlen_q=max(kv_lens), max_seqlen_k=max(kv_lens), softmax_scale=d**-0.5, causal=True,
    )
    assert_bitwise(packed, prefill, "packed vs paged prefill")
    off = 0
    for s, n in enumerate(kv_lens):
        assert_bitwise(prefill[off + n - 1], decode[s], f"prefill last row vs decode (seq {s})")
        off += n
    # chunked prefill: the last 5 rows computed as a 5-token chunk on a cached prefix
    chunk = _run_paged([x[-5:] for x in qp], k, v, page)
    off = 0
    for s, n in enumerate(kv_lens):
        assert_bitwise(prefill[off + n - 5 : off + n], chunk[5 * s : 5 * s + 5], f"chunk rows (seq {s})")
        off += n


def test_single_key_returns_value_exactly():
    q, k, v = _seqs([1, 1], 4, 32, 10), _seqs([1, 1], 2, 32, 11), _seqs([1, 1], 2, 32, 12)
    out = _run_paged(q, k, v, 16)
    ref = torch.cat([x.repeat_interleave(2, dim=1) for x in v])
    assert_bitwise(out, ref, "softmax over one key")


def test_mla_head_dims_match_eager():
    kv_lens, q_lens = [40, 70], [40, 1]
    q, k, v = _seqs(q_lens, 16, 192, 13, 0.1), _seqs(kv_lens, 16, 192, 14, 0.1), _seqs(kv_lens, 16, 128, 15, 0.1)
    out = _run_paged(q, k, v, 16)
    assert out.shape == (41, 16, 128)
    ref = torch.cat([OA.eager_attention(a, b, c, 192**-0.5) for a, b, c in zip(q, k, v)], dim=0)
    torch.testing.assert_close(out.cpu(), ref, atol=3e-3, rtol=3e-3)


def test_config2_shaped_decode_subset():
    # config 2 geometry (16q / 8kv / 128, page 16, shuffled pages) on 6 sequences
    g = torch.Generator().manual_seed(2)
    kv_lens = torch.randint(128, 4097, (6,), generator=g).tolist()
    q, k, v = _seqs([1] * 6, 16, 128, 16), _seqs(kv_lens, 8, 128, 17), _seqs(kv_lens, 8, 128, 18)
    pages = sum((n + 15) // 16 for n in kv_lens)
    perm = torch.randperm(pages + 50, generator=g)
    k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, 16, perm=perm, extra_pages=50)
    cu = _cu([1] * 6)
    used = torch.tensor(kv_lens, dtype=torch.int32)
    out, _ = flash_attn_varlen_func(torch.cat(q).cuda(), k_cache.cuda(), v_cache.cuda(), cu_seqlens_q=cu.cuda(),
                                    max_seqlen_q=1, seqused_k=used.cuda(), page_table=table.cuda(), causal=True)
    ref = OA.paged_attention_ref(torch.cat(q), k_cache, v_cache, cu, used, table, 128**-0.5)
    assert_bf16_close(out, ref, max_ulp=2, atol_frac=2e-3, what="config-2 decode vs eager oracle")
    for s in range(6):
        one, _ = flash_attn_varlen_func(q[s].cuda(), k_cache.cuda(), v_cache.cuda(), cu_seqlens_q=_cu([1]).cuda(),
                                        max_seqlen_q=1, seqused_k=used[s : s + 1].cuda(),
                                        page_table=table[s : s + 1].cuda(), causal=True)
        assert_bitwise(one[0], out[s], f"sequence {s} alone on the same pages")


def test_store_kvcache_exact_and_skips():
    g = torch.Generator().manual_seed(19)
    for dk, dv in ((128, 128), (192, 128)):
        key = torch.randn(37, 4, dk, generator=g).to(torch.bfloat16)
        val = torch.randn(37, 4, dv, generator=g).to(torch.bfloat16)
        kc = torch.randn(8, 16, 4, dk, generator=g).to(torch.bfloat16)
        vc = torch.randn(8, 16, 4, dv, generator=g).to(torch.bfloat16)
        slots = torch.randperm(128, generator=g)[:37].to(torch.int32)
        slots[[3, 11]] = -1
        kc_ref, vc_ref = kc.clone(), vc.clone()
        OA.store_kvcache_ref(key, val, kc_ref, vc_ref, slots)
        kg, vg = kc.cuda(), vc.cuda()
        store_kvcache(key.cuda(), val.cuda(), kg, vg, slots.cuda())
        assert_bitwise(kg, kc_ref, "key cache")
        assert_bitwise(vg, vc_ref, "value cache")


def test_attention_wrapper_shape_and_cache_write():
    qh, kh, d, page = 4, 2, 32, 16
    q_lens, past = [3, 1], [5, 20]
    kv_lens = [p + n for p, n in zip(past, q_lens)]
    q, k, v = _seqs(q_lens, qh, d, 20, 0.1), _seqs(kv_lens, kh, d, 21, 0.1), _seqs(kv_lens, kh, d, 22, 0.1)
    # cache holds only the past; the wrapper must write the new tokens
    k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, page)
    slots, newk, newv = [], [], []
    for s, (p, n) in enumerate(zip(past, q_lens)):
        for pos in range(p, p + n):
            slots.append(int(table[s, pos // page]) * page + pos % page)
            k_cache.view(-1, kh, d)[slots[-1]] = 0
            v_cache.view(-1, kh, d)[slots[-1]] = 0
        newk.append(k[s][p:])
        newv.append(v[s][p:])
    kc, vc = k_cache.cuda(), v_cache.cuda()
    set_kv_cache_context(
        is_paged_attn=True, key_cache={0: kc}, value_cache={0: vc}, block_tables=table.cuda(),
        context_lens=torch.tensor(kv_lens, dtype=torch.int32).cuda(),
        slot_mapping=torch.tensor(slots, dtype=torch.int32).cuda(), query_start_loc=_cu(q_lens).cuda(), max_seqlen_q=3,
    )
    try:
        module = torch.nn.Module()
        module.layer_idx = 0
        qq = torch.cat(q).transpose(0, 1).unsqueeze(0).cuda()
        kk = torch.cat(newk).transpose(0, 1).unsqueeze(0).cuda()
        vv = torch.cat(newv).transpose(0, 1).unsqueeze(0).cuda()
        out, aux = flash_attention_forward(module, qq, kk, vv, None, scaling=d**-0.5)
    finally:
        clear_kv_cache_context()
    assert aux is None and out.shape == (4, qh, d)
    ref = torch.cat([OA.eager_attention(a, b, c, d**-0.5) for a, b, c in zip(q, k, v)], dim=0)
    torch.testing.assert_close(out.cpu(), ref, atol=3e-3, rtol=3e-3)
    full_k, _, _ = OA.make_paged_kv_cache(k, v, page)
    assert_bitwise(kc, full_k, "wrapper wrote the new keys")


def test_head_major_cache_views_store_and_attend_like_the_reference_layout():
    # KVCacheStore(head_major=True) hands out [blocks, page, heads, D] views of [blocks, heads, page, D] memory:
    # the scatter writes the same elements (slot -1 skipped) and the wrapper's attention gives the same bits
    import types

    from vexact_amd.batch_invariant_ops.kv_cache_context import KVCacheStore

    qh, kh, d, page = 8, 2, 128, 16
    q_lens, past = [3, 1, 40, 1], [5, 200, 0, 77]
    kv_lens = [p + n for p, n in zip(past, q_lens)]
    q, k, v = _seqs(q_lens, qh, d, 60, 0.1), _seqs(kv_lens, kh, d, 61, 0.1), _seqs(kv_lens, kh, d, 62, 0.1)
    k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, page)
    slots, newk, newv = [], [], []
    for s, (p, n) in enumerate(zip(past, q_lens)):
        for pos in range(p, p + n):
            slots.append(int(table[s, pos // page]) * page + pos % page)
            k_cache.view(-1, kh, d)[slots[-1]] = 0
            v_cache.view(-1, kh, d)[slots[-1]] = 0
        newk.append(k[s][p:])
        newv.append(v[s][p:])
    slots[1] = -1  # one token that must not be written (its zeroed slot stays zero in both layouts)
    hf_cfg = types.SimpleNamespace(num_hidden_layers=1, num_key_value_heads=kh, head_dim=d, hidden_size=qh * d,
                                   num_attention_heads=qh, dtype=torch.bfloat16)
    cache_cfg = types.SimpleNamespace(page_size=page, max_cache_blocks=k_cache.shape[0])
    outs, caches = [], []
    for head_major in (False, True):
        store = KVCacheStore(hf_cfg, cache_cfg, torch.device("cuda"), head_major=head_major)
        kc, vc = store.key_cache[0], store.value_cache[0]
        assert kc.shape == k_cache.shape and kc.is_contiguous() != head_major
        kc.copy_(k_cache.cuda())
        vc.copy_(v_cache.cuda())
        set_kv_cache_context(
            is_paged_attn=True, key_cache=store.key_cache, value_cache=store.value_cache, block_tables=table.cuda(),
            context_lens=torch.tensor(kv_lens, dtype=torch.int32).cuda(),
            slot_mapping=torch.tensor(slots, dtype=torch.int32).cuda(), query_start_loc=_cu(q_lens).cuda(), max_seqlen_q=40,
        )
        try:
            module = torch.nn.Module()
            module.layer_idx = 0
            qq = torch.cat(q).transpose(0, 1).unsqueeze(0).cuda()
            kk = torch.cat(newk).transpose(0, 1).unsqueeze(0).cuda()
            vv = torch.cat(newv).transpose(0, 1).unsqueeze(0).cuda()
            out, _ = flash_attention_forward(module, qq, kk, vv, None, scaling=d**-0.5)
        finally:
            clear_kv_cache_context()
        outs.append(out.clone())
        caches.append((kc.contiguous().clone(), vc.contiguous().clone()))
    assert_bitwise(outs[1], outs[0], "attention output: head-major cache views vs the reference layout")
    assert_bitwise(caches[1][0], caches[0][0], "keys written through the strided scatter")
    assert_bitwise(caches[1][1], caches[0][1], "values written through the strided scatter")
    assert float(caches[0][0].view(-1, kh, d)[slots[0]].abs().sum()) > 0 and float(caches[1][0].view(-1, kh, d)[slots[2]].abs().sum()) > 0


def test_attention_wrapper_gives_the_same_bits_for_any_memory_layout():
    # HuggingFace hands [1, heads, tokens, dim] tensors that are views of [1, tokens, heads, dim] memory; the wrapper
    # reads them through strides. A tensor that really is head-major in memory must give the same bits, in the
    # paged, the packed-context and the no-context branch.
    qh, kh, d, page = 8, 2, 128, 16
    lens = [37, 5, 64]
    q, k, v = _seqs(lens, qh, d, 40), _seqs(lens, kh, d, 41), _seqs(lens, kh, d, 42)
    T = sum(lens)
    cu = _cu(lens).cuda()
    module = torch.nn.Module()
    module.layer_idx = 0
    module.is_causal = True

    def views(layout):
        outs = []
        for t in (torch.cat(q), torch.cat(k), torch.cat(v)):
            x = t.cuda()                                        # [T, H, D] in memory
            if layout == "token-major":
                outs.append(x.transpose(0, 1).unsqueeze(0))     # [1, H, T, D] view of it
            else:
                outs.append(x.transpose(0, 1).contiguous().unsqueeze(0))  # [1, H, T, D] in memory
        return outs

    results = {}
    for layout in ("token-major", "head-major"):
        qq, kk, vv = views(layout)
        # paged: empty cache, every token of the step is written, then attended
        k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, page)
        kc, vc = torch.zeros_like(k_cache).cuda(), torch.zeros_like(v_cache).cuda()
        slots = [int(table[s, pos // page]) * page + pos % page for s, n in enumerate(lens) for pos in range(n)]
        set_kv_cache_context(is_paged_attn=True, key_cache={0: kc}, value_cache={0: vc}, block_tables=table.cuda(),
                             context_lens=torch.tensor(lens, dtype=torch.int32).cuda(),
                             slot_mapping=torch.tensor(slots, dtype=torch.int32).cuda(), query_start_loc=cu, max_seqlen_q=max(lens))
        try:
            paged, _ = flash_attention_forward(module, qq, kk, vv, None, scaling=d**-0.5)
        finally:
            clear_kv_cache_context()
        assert_bitwise(kc, k_cache, f"{layout}: keys written by the wrapper")
        # packed context
        set_kv_cache_context(is_paged_attn=False, context_lens=torch.tensor(lens, dtype=torch.int32).cuda(),
                             query_start_loc=cu, max_seqlen_q=max(lens))
        try:
            packed, _ = flash_attention_forward(module, qq, kk, vv, None, scaling=d**-0.5)
        finally:
            clear_kv_cache_context()
        # no context: boundaries in the call
        plain, _ = flash_attention_forward(module, qq, kk, vv, None, scaling=d**-0.5, cu_seq_lens_q=cu, cu_seq_lens_k=cu,
                                           max_length_q=max(lens), max_length_k=max(lens))
        assert paged.shape == (T, qh, d) and packed.shape == (T, qh, d) and plain.shape == (1, T, qh, d)
        assert_bitwise(packed, paged, f"{layout}: packed context vs paged")
        assert_bitwise(plain[0], paged, f"{layout}: no context vs paged")
        results[layout] = paged
    assert_bitwise(results["head-major"], results["token-major"], "head-major vs token-major inputs")
    ref = torch.cat([OA.eager_attention(a, b, c, d**-0.5) for a, b, c in zip(q, k, v)], dim=0)
    assert_bf16_close(results["token-major"], ref, max_ulp=2, atol_frac=2e-3, what="wrapper vs eager oracle")


def test_rows_of_a_sequence_without_any_key_are_left_alone():
    # a sequence that has a query token but seqused_k = 0 (never built by the model runner): its output row is not
    # written by any kernel form, and the other sequences are not disturbed
    from vexact_amd import ops

    qh, kh, d, page = 4, 2, 128, 16
    kv_lens = [40, 0, 300]
    k, v = _seqs([40, 1, 300], kh, d, 51), _seqs([40, 1, 300], kh, d, 52)
    q = _seqs([1, 1, 1], qh, d, 50)
    k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, page)
    used = torch.tensor(kv_lens, dtype=torch.int32).cuda()
    cu = _cu([1, 1, 1]).cuda()
    ref = [OA.eager_attention(q[s], k[s], v[s], d**-0.5) for s in (0, 2)]
    for max_q, kernel in ((1, "split"), (1, "fused"), (2, "auto")):
        out = torch.full((3, qh, d), 9.0, dtype=torch.bfloat16, device="cuda")
        ops.paged_attention(torch.cat(q).cuda(), k_cache.cuda(), v_cache.cuda(), cu, used, table.cuda(), d**-0.5, max_q,
                            out=out, decode_kernel=kernel)
        assert bool((out[1] == 9.0).all()), f"{kernel}: the row without keys was written"
        for row, want in ((0, ref[0]), (2, ref[1])):  # the neighbours are undisturbed (precision is tested elsewhere)
            assert float((out[row: row + 1].cpu().float() - want.float()).abs().max()) <= 1e-2, f"{kernel}: sequence {row}"


def test_argument_errors():
    q, k, v = _seqs([2], 4, 32, 23), _seqs([2], 2, 32, 24), _seqs([2], 2, 32, 25)
    qg, kg, vg = q[0].cuda(), k[0].cuda(), v[0].cuda()
    cu = _cu([2]).cuda()
    with pytest.raises(ValueError, match="max_seqlen_k is required"):
        flash_attn_varlen_func(qg, kg, vg, cu_seqlens_q=cu, cu_seqlens_k=cu, max_seqlen_q=2, causal=True)
    with pytest.raises(ValueError, match="max_seqlen_q is required"):
        flash_attn_varlen_func(qg, kg, vg, cu_seqlens_q=cu, cu_seqlens_k=cu, max_seqlen_k=2, causal=True)
    k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, 16)
    used = torch.tensor([2], dtype=torch.int32).cuda()
    with pytest.raises(ValueError, match="pass only one of page_table or block_table"):
        flash_attn_varlen_func(qg, k_cache.cuda(), v_cache.cuda(), cu_seqlens_q=cu, seqused_k=used,
                               page_table=table.cuda(), block_table=table.cuda(), causal=True)
    with pytest.raises(NotImplementedError):
        flash_attn_varlen_func(qg, kg, vg, cu_seqlens_q=cu, cu_seqlens_k=cu, max_seqlen_q=2, max_seqlen_k=2, dropout_p=0.1)
    with pytest.raises(NotImplementedError):
        flash_attn_varlen_func(qg, kg, vg, cu_seqlens_q=cu, cu_seqlens_k=cu, max_seqlen_q=2, max_seqlen_k=2, softcap=1.0)
    with pytest.raises(NotImplementedError):
        flash_attn_varlen_func(qg, kg, vg, cu_seqlens_q=cu, cu_seqlens_k=cu, max_seqlen_q=2, max_seqlen_k=2, window_size=(4, 0))
    with pytest.raises(NotImplementedError, match="only supports causal=True"):
        flash_attn_varlen_func(qg, k_cache.cuda(), v_cache.cuda(), cu_seqlens_q=cu, seqused_k=used,
                               page_table=table.cuda(), causal=False)
    with pytest.raises(ValueError, match="torch.int32"):
        flash_attn_varlen_func(qg, k_cache.cuda(), v_cache.cuda(), cu_seqlens_q=cu.long(), seqused_k=used,
                               page_table=table.cuda(), causal=True)


def test_paged_backward_raises():
    q, k, v = _seqs([2], 4, 32, 26), _seqs([2], 2, 32, 27), _seqs([2], 2, 32, 28)
    k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, 16)
    qg = q[0].cuda().requires_grad_(True)
    out, _ = flash_attn_varlen_func(qg, k_cache.cuda(), v_cache.cuda(), cu_seqlens_q=_cu([2]).cuda(),
                                    seqused_k=torch.tensor([2], dtype=torch.int32).cuda(), page_table=table.cuda(),
                                    causal=True, max_seqlen_q=2)
    with pytest.raises(NotImplementedError, match="paged triton flash_attn_varlen_func backward"):
        out.sum().backward()


def test_packed_non_causal_matches_eager():
    q, k, v = _seqs([5, 9], 4, 64, 29, 0.2), _seqs([12, 9], 2, 64, 30, 0.2), _seqs([12, 9], 2, 64, 31, 0.2)
    out, _ = flash_attn_varlen_func(torch.cat(q).cuda(), torch.cat(k).cuda(), torch.cat(v).cuda(),
                                    cu_seqlens_q=_cu([5, 9]).cuda(), cu_seqlens_k=_cu([12, 9]).cuda(),
                                    max_seqlen_q=9, max_seqlen_k=12, causal=False)
    ref = torch.cat([OA.eager_attention(a, b, c, 64**-0.5, causal=False) for a, b, c in zip(q, k, v)])
    torch.testing.assert_close(out.cpu(), ref, atol=3e-3, rtol=3e-3)


@pytest.mark.parametrize(
    ("qh", "kh", "dk", "dv", "page", "head_major"),
    [(32, 4, 128, 128, 16, True), (8, 8, 64, 64, 16, False), (48, 2, 128, 128, 32, False), (16, 1, 192, 128, 16, False),
     (4, 2, 32, 32, 24, False)],
)
def test_decode_forms_agree_bitwise(qh, kh, dk, dv, page, head_major):
    """One wavefront per chunk + combine launch vs chunks folded inside the workgroup: same bits, for
    lengths around the 256-key chunk edges, 1..9 chunks, GQA groups of 1 / 8 / 16 / 24 heads, a page
    size that is not a power of two, and the head-major physical cache layout."""
    from vexact_amd import ops

    kv_lens = [1, 63, 64, 255, 256, 257, 511, 513, 1024, 1025, 1300, 2047, 2048, 2049, 700, 40]
    g = torch.Generator().manual_seed(11)
    k = [(torch.randn(n, kh, dk, generator=g) * 0.3).to(torch.bfloat16) for n in kv_lens]
    v = [(torch.randn(n, kh, dv, generator=g) * 0.3).to(torch.bfloat16) for n in kv_lens]
    q = (torch.randn(len(kv_lens), qh, dk, generator=g) * 0.3).to(torch.bfloat16).cuda()
    perm = torch.randperm(sum((n + page - 1) // page for n in kv_lens), generator=g)
    k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, page, perm=perm)
    kc, vc = k_cache.cuda(), v_cache.cuda()
    if head_major:
        kc = kc.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
        vc = vc.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    cu = torch.arange(len(kv_lens) + 1, dtype=torch.int32).cuda()
    used = torch.tensor(kv_lens, dtype=torch.int32).cuda()
    outs = {kind: ops.paged_attention(q, kc, vc, cu, used, table.cuda(), dk**-0.5, 1, decode_kernel=kind)
            for kind in ("split", "fused", "auto")}
    assert_bitwise(outs["fused"], outs["split"], "fused vs split decode")
    assert_bitwise(outs["auto"], outs["split"], "auto vs split decode")
    # the order in which the workgroups take the sequences (longest first) does not change a bit
    order = torch.tensor(sorted(range(len(kv_lens)), key=lambda i: (-kv_lens[i], i)), dtype=torch.int32).cuda()
    for kind in ("split", "fused"):
        assert_bitwise(ops.paged_attention(q, kc, vc, cu, used, table.cuda(), dk**-0.5, 1, decode_kernel=kind, seq_order=order),
                       outs["split"], f"{kind} decode with a sequence order")
    ref = torch.stack([OA.eager_attention(q[i : i + 1].cpu(), k[i], v[i], dk**-0.5)[0] for i in range(len(kv_lens))])
    torch.testing.assert_close(outs["fused"].cpu(), ref, atol=3e-3, rtol=3e-3)


def _packed_fwd_bwd(q_seqs, k_seqs, v_seqs, do_seqs):
    q = torch.cat(q_seqs).cuda().requires_grad_()
    k = torch.cat(k_seqs).cuda().requires_grad_()
    v = torch.cat(v_seqs).cuda().requires_grad_()
    q_lens, kv_lens = [t.shape[0] for t in q_seqs], [t.shape[0] for t in k_seqs]
    out, _ = flash_attn_varlen_func(q, k, v, cu_seqlens_q=_cu(q_lens).cuda(), cu_seqlens_k=_cu(kv_lens).cuda(),
                                    max_seqlen_q=max(q_lens), max_seqlen_k=max(kv_lens), causal=True)
    out.backward(torch.cat(do_seqs).cuda())
    return out.detach().cpu(), q.grad.cpu(), k.grad.cpu(), v.grad.cpu()


@pytest.mark.parametrize(("qh", "kh", "d", "q_lens", "kv_lens"), [
    (8, 2, 128, [24, 19], [24, 19]),
    (4, 4, 64, [70, 1, 33], [70, 90, 33]),
    (8, 1, 128, [130, 5, 64, 1], [130, 200, 64, 65]),
    (6, 2, 64, [17], [300]),
])
def test_packed_backward_matches_autograd_and_is_batch_invariant(qh, kh, d, q_lens, kv_lens):
    # formulas of the reference's backward kernels (triton_invariant_attention.py:193-430) against
    # autograd through an fp32 eager attention; P and dS are rounded to bf16 on the GPU
    print(f"[case] attention backward Hq={qh} Hkv={kh} D={d} q={q_lens} kv={kv_lens}", flush=True)
    q_seqs, k_seqs, v_seqs = _seqs(q_lens, qh, d, 1), _seqs(kv_lens, kh, d, 2), _seqs(kv_lens, kh, d, 3)
    do_seqs = _seqs(q_lens, qh, d, 4)
    out, dq, dk, dv = _packed_fwd_bwd(q_seqs, k_seqs, v_seqs, do_seqs)
    scale = d ** -0.5
    o = 0
    ok = 0
    for s, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        qf, kf, vf = (t.float().requires_grad_() for t in (q_seqs[s], k_seqs[s], v_seqs[s]))
        g = qh // kh
        kk, vv = kf.repeat_interleave(g, dim=1), vf.repeat_interleave(g, dim=1)
        sc = torch.einsum("qhd,khd->hqk", qf, kk) * scale
        pos = torch.arange(ql) + (kl - ql)
        mask = torch.arange(kl)[None, :] <= pos[:, None]
        sc = sc.masked_fill(~mask[None], float("-inf"))
        ref = torch.einsum("hqk,khd->qhd", torch.softmax(sc, -1), vv)
        ref.backward(do_seqs[s].float())
        for name, got, want in (("dq", dq[o : o + ql], qf.grad), ("dk", dk[ok : ok + kl], kf.grad), ("dv", dv[ok : ok + kl], vf.grad)):
            err = (got.float() - want).abs()
            tol = 2e-2 * float(want.abs().max())
            assert float(err.max()) <= tol, f"{name} of sequence {s}: max err {float(err.max()):.4f} > {tol:.4f}"
            assert float(err.mean()) <= 2e-3 * float(want.abs().max()), f"{name} of sequence {s}: mean err"
        assert_bf16_close(out[o : o + ql], ref.detach().to(torch.bfloat16), max_ulp=2, atol_frac=3e-3, what=f"out of sequence {s}")
        # and against the restatement with the same bf16 roundings of P and dS (tighter)
        odq, odk, odv = OA.attention_backward_ref(q_seqs[s], k_seqs[s], v_seqs[s], do_seqs[s], scale)
        for name, got, want in (("dq", dq[o : o + ql], odq), ("dk", dk[ok : ok + kl], odk), ("dv", dv[ok : ok + kl], odv)):
            err = (got.float() - want.float()).abs()
            top = float(want.float().abs().max())
            assert float(err.max()) <= 1e-2 * top and float(err.mean()) <= 1e-3 * top, (
                f"{name} of sequence {s} vs the CPU restatement: max {float(err.max()):.4g}, mean {float(err.mean()):.4g}, scale {top:.4g}")
        # the sequence alone gives the same gradient bits
        _, dq1, dk1, dv1 = _packed_fwd_bwd(q_seqs[s : s + 1], k_seqs[s : s + 1], v_seqs[s : s + 1], do_seqs[s : s + 1])
        assert_bitwise(dq1, dq[o : o + ql], f"dq of sequence {s} alone vs in the batch")
        assert_bitwise(dk1, dk[ok : ok + kl], f"dk of sequence {s} alone vs in the batch")
        assert_bitwise(dv1, dv[ok : ok + kl], f"dv of sequence {s} alone vs in the batch")
        o += ql
        ok += kl


def test_packed_forward_with_lse_keeps_the_output_bits():
    from vexact_amd import ops
    q_lens, kv_lens = [40, 3, 129], [40, 77, 129]
    q, k, v = (torch.cat(_seqs(l, h, 128, sd)).cuda() for l, h, sd in ((q_lens, 8, 1), (kv_lens, 2, 2), (kv_lens, 2, 3)))
    cu_q, cu_k = _cu(q_lens).cuda(), _cu(kv_lens).cuda()
    plain = ops.packed_attention(q, k, v, cu_q, cu_k, 128 ** -0.5, True, max(q_lens))
    out, lse = ops.packed_attention(q, k, v, cu_q, cu_k, 128 ** -0.5, True, max(q_lens), return_lse=True)
    assert_bitwise(out, plain, "output with and without the log-sum-exp")
    o = ok = 0
    for ql, kl in zip(q_lens, kv_lens):
        sc = torch.einsum("qhd,khd->hqk", q[o : o + ql].float().cpu(), k[ok : ok + kl].float().cpu().repeat_interleave(4, dim=1)) * 128 ** -0.5
        mask = torch.arange(kl)[None, :] <= (torch.arange(ql) + (kl - ql))[:, None]
        want = torch.logsumexp(sc.masked_fill(~mask[None], float("-inf")), -1).transpose(0, 1)
        assert float((lse[o : o + ql].cpu() - want).abs().max()) < 2e-3
        o += ql
        ok += kl


def test_decode_forms_agree_bitwise_with_many_workgroups():
    """256 sequences x 4 kv heads = 1024 workgroups: the fused kernel then runs with 4 wavefronts per
    workgroup (several rounds for the longer sequences); same bits as one wavefront per chunk."""
    from vexact_amd import ops

    g = torch.Generator().manual_seed(21)
    kv_lens = torch.randint(1, 1500, (256,), generator=g).tolist()
    kv_lens[:4] = [2049, 1, 256, 1025]
    k = [(torch.randn(n, 4, 128, generator=g) * 0.3).to(torch.bfloat16) for n in kv_lens]
    v = [(torch.randn(n, 4, 128, generator=g) * 0.3).to(torch.bfloat16) for n in kv_lens]
    q = (torch.randn(len(kv_lens), 32, 128, generator=g) * 0.3).to(torch.bfloat16).cuda()
    k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, 16)
    kc, vc = k_cache.cuda(), v_cache.cuda()
    cu = torch.arange(len(kv_lens) + 1, dtype=torch.int32).cuda()
    used = torch.tensor(kv_lens, dtype=torch.int32).cuda()
    order = torch.tensor(sorted(range(len(kv_lens)), key=lambda i: (-kv_lens[i], i)), dtype=torch.int32).cuda()
    split = ops.paged_attention(q, kc, vc, cu, used, table.cuda(), 128**-0.5, 1, decode_kernel="split")
    for kw in (dict(decode_kernel="fused"), dict(decode_kernel="auto"), dict(decode_kernel="fused", seq_order=order)):
        assert_bitwise(ops.paged_attention(q, kc, vc, cu, used, table.cuda(), 128**-0.5, 1, **kw), split, str(kw))
    for i in (0, 1, 2, 3, 100):
        ref = OA.eager_attention(q[i : i + 1].cpu(), k[i], v[i], 128**-0.5)[0]
        torch.testing.assert_close(split[i].cpu(), ref, atol=3e-3, rtol=3e-3)
