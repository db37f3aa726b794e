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
from tests.util import assert_bf16_close, assert_bitwise

pytestmark = pytest.mark.gpu

from vexact_amd import ops  # noqa: E402
from vexact_amd.batch_invariant_ops import triton_flash_attn_varlen_func as flash_attn_varlen_func  # noqa: E402
from vexact_amd.batch_invariant_ops.fused_moe import fused_moe_forward  # noqa: E402


def _cu(lens):
    return torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)


def _bf16_normal(shape, seed):
    """Drawn on the GPU (the CPU generator would take minutes at these sizes); the CPU copy has the same bits."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    t = torch.empty(shape, dtype=torch.bfloat16, device="cuda")
    t.normal_(0.0, 1.0, generator=g)
    return t


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
    for s in (0, 1, 5):
        ks = OA.gather_paged(kc, table[s], kv_lens[s])
        vs = OA.gather_paged(vc, table[s], kv_lens[s])
        for i in (0, 255, C - 1):
            n = int(prefix[s]) + i + 1
            ref = OA.eager_attention(qc[s * C + i : s * C + i + 1], ks[:n], vs[:n], D**-0.5)
            torch.testing.assert_close(out[s * C + i : s * C + i + 1].cpu().float(), ref.float(), atol=3e-3, rtol=3e-3,
                                       msg=lambda m: f"sequence {s} chunk row {i} vs eager oracle: {m}")


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
    assert_bf16_close(full[rows.cuda()], ref, max_ulp=2, atol_frac=2e-3, what="config-4 rows vs fused-order oracle")
