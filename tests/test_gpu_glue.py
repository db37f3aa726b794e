"""GPU parity of the glue kernels between the q/k/v projection and attention, on their own:
``vx_qk_norm_rope_store`` (per-head RMSNorm of q and k with DISTINCT non-unit weights, rotary embedding at
large positions, cache write at slot_mapping incl. slot -1, contiguous and head-major caches) and
``vx_embedding``, against the CPU oracle, which builds its own cos / sin tables from rope_theta.
Follows the HuggingFace attention front end the reference patches and the reference's cache write
(vexact/batch_invariant_ops/triton_invariant_attention.py:1047-1054, kv_cache_context.py:294-314)."""

import numpy as np
import pytest
import torch

from oracle import decoder as OD
from tests.util import assert_bitwise, bf16_ulp_distance

BF = torch.bfloat16


def test_product_rope_tables_equal_the_oracle_tables():
    # CPU-only: the table builder the decoder uses against the oracle's (which is pinned to HuggingFace's)
    from vexact_amd.decoder import DecoderConfig, rope_tables

    for theta, D, n in ((1.0e6, 128, 40960), (1.0e4, 64, 2048)):
        cfg = DecoderConfig(head_dim=D, rope_theta=theta, max_model_len=n)
        cos, sin = rope_tables(cfg, "cpu")
        cos_ref, sin_ref = OD.rope_tables_ref(D, theta, n)
        assert_bitwise(cos, cos_ref, "cos table")
        assert_bitwise(sin, sin_ref, "sin table")


def _case(seed, T, Hq, Hkv, D, max_pos, theta, page, blocks):
    g = torch.Generator().manual_seed(seed)
    qkv = (torch.randn(T, (Hq + 2 * Hkv) * D, generator=g) * 1.7).to(BF)
    qw = (0.5 + torch.rand(D, generator=g)).to(BF)
    kw = (0.5 + torch.rand(D, generator=g)).to(BF)
    pos = torch.randint(0, max_pos, (T,), generator=g)
    pos[0], pos[-1] = 0, max_pos - 1
    slots = torch.randperm(blocks * page, generator=g)[:T].to(torch.int32)
    slots[torch.arange(T) % 5 == 3] = -1
    cos, sin = OD.rope_tables_ref(D, theta, max_pos)
    return qkv, qw, kw, pos, slots, cos, sin


@pytest.mark.gpu
@pytest.mark.parametrize("D,Hq,Hkv,T,max_pos,theta,pos_dtype,head_major", [
    (128, 8, 2, 300, 40960, 1.0e6, torch.int64, False),
    (128, 32, 4, 257, 40960, 1.0e6, torch.int32, True),
    (64, 4, 4, 33, 8192, 1.0e4, torch.int64, True),
    (128, 4, 1, 1, 4096, 1.0e6, torch.int32, False),
])
def test_qk_norm_rope_store_matches_oracle(D, Hq, Hkv, T, max_pos, theta, pos_dtype, head_major):
    from vexact_amd import ops

    page, blocks = 16, (T + 15) // 16 + 3
    qkv, qw, kw, pos, slots, cos, sin = _case(7, T, Hq, Hkv, D, max_pos, theta, page, blocks)
    # oracle
    kc_ref = torch.zeros(blocks, page, Hkv, D, dtype=BF)
    vc_ref = torch.zeros_like(kc_ref)
    q_ref, k_ref = OD.qk_norm_rope_store_ref(qkv, qw, kw, cos, sin, pos, slots, kc_ref, vc_ref, Hq, Hkv, D)
    # kernel: caches pre-filled with a marker so that untouched rows are seen to be untouched
    def cache():
        if head_major:
            return torch.full((blocks, Hkv, page, D), 7.0, dtype=BF, device="cuda").permute(0, 2, 1, 3)
        return torch.full((blocks, page, Hkv, D), 7.0, dtype=BF, device="cuda")
    kc, vc = cache(), cache()
    q = torch.empty(T, Hq, D, dtype=BF, device="cuda")
    k_out = torch.empty(T, Hkv, D, dtype=BF, device="cuda")
    ops.qk_norm_rope_store(qkv.cuda(), qw.cuda(), kw.cuda(), cos.cuda(), sin.cuda(), pos.to(pos_dtype).cuda(), slots.cuda(),
                           q, kc, vc, Hq, Hkv, D, 1e-6, k_out=k_out)
    torch.cuda.synchronize()
    q, k_out, kc, vc = q.cpu(), k_out.cpu(), kc.cpu().contiguous(), vc.cpu().contiguous()
    # the kernel divides by sqrt where the oracle multiplies by rsqrt: now and then one bf16 ulp on the normalised
    # value, hence at most 2 on the sum of the two rotated products (measured: 1 or 2 elements of 10^6 differ)
    for name, got, want in (("q", q, q_ref), ("k", k_out, k_ref)):
        ulp = bf16_ulp_distance(got, want)
        absd = (got.float() - want.float()).abs()
        small = absd <= 2.0 ** -7 * want.float().abs().clamp(min=2.0 ** -6)  # cancellation in a*cos + b*sin
        print(f"{name}: {float((ulp == 0).float().mean()):.4f} exact, {float((ulp <= 1).float().mean()):.4f} within 1 ulp, "
              f"worst {int(ulp.max())} ulp")
        assert bool(((ulp <= 2) | small).all()), f"{name}: beyond 2 bf16 ulp"
        assert float((ulp == 0).float().mean()) >= 0.999, f"{name}: too few exact elements"
    # cache rows: the written K row is the kernel's own k output bit for bit, V is a plain copy, rows of slot -1
    # and rows no token maps to keep the marker
    flat_k, flat_v = kc.view(-1, Hkv, D), vc.view(-1, Hkv, D)
    v_src = qkv[:, (Hq + Hkv) * D:].view(T, Hkv, D)
    keep = torch.ones(flat_k.shape[0], dtype=torch.bool)
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        keep[s] = False
        assert torch.equal(flat_k[s], k_out[t]), f"key row of token {t}"
        assert torch.equal(flat_v[s], v_src[t]), f"value row of token {t}"
    assert bool((flat_k[keep] == 7.0).all()) and bool((flat_v[keep] == 7.0).all()), "a row without a slot was written"
    assert_bitwise(flat_v[~keep], vc_ref.view(-1, Hkv, D)[~keep], "value cache vs oracle")
    # teeth: with the two norm weights swapped the oracle is far away
    q_sw, _ = OD.qk_norm_rope_store_ref(qkv, kw, qw, cos, sin, pos, slots, None, None, Hq, Hkv, D)
    assert float((bf16_ulp_distance(q, q_sw) > 2).float().mean()) > 0.5


@pytest.mark.gpu
def test_qk_norm_rope_store_rows_do_not_depend_on_the_batch():
    from vexact_amd import ops

    D, Hq, Hkv, T = 128, 8, 2, 64
    qkv, qw, kw, pos, slots, cos, sin = _case(9, T, Hq, Hkv, D, 40960, 1.0e6, 16, 8)
    dev = [t.cuda() for t in (qkv, qw, kw, cos, sin, pos)]
    def run(rows):
        q = torch.empty(len(rows), Hq, D, dtype=BF, device="cuda")
        k = torch.empty(len(rows), Hkv, D, dtype=BF, device="cuda")
        ops.qk_norm_rope_store(dev[0][rows].contiguous(), dev[1], dev[2], dev[3], dev[4], dev[5][rows].contiguous(), None,
                               q, None, None, Hq, Hkv, D, 1e-6, k_out=k)
        return q.cpu(), k.cpu()
    q_all, k_all = run(torch.arange(T))
    for r in (0, 17, 63):
        q1, k1 = run(torch.tensor([r]))
        assert_bitwise(q1, q_all[r: r + 1], f"q row {r}")
        assert_bitwise(k1, k_all[r: r + 1], f"k row {r}")


@pytest.mark.gpu
@pytest.mark.parametrize("id_dtype", [torch.int32, torch.int64])
def test_embedding_is_a_row_gather(id_dtype):
    from vexact_amd import ops

    g = torch.Generator().manual_seed(3)
    table = torch.randn(1000, 256, generator=g).to(BF)
    ids = torch.randint(0, 1000, (77,), generator=g)
    ids[0], ids[1], ids[2] = 0, 999, 999
    out = ops.embedding(table.cuda(), ids.to(id_dtype).cuda())
    assert_bitwise(out.cpu(), OD.embedding_ref(table, ids), "embedding rows")
    # into a caller's buffer, at the full model width
    table = torch.randn(4096, 2048, generator=g).to(BF)
    ids = torch.from_numpy(np.random.default_rng(4).integers(0, 4096, size=256))
    buf = torch.zeros(256, 2048, dtype=BF, device="cuda")
    ops.embedding(table.cuda(), ids.to(id_dtype).cuda(), out=buf)
    assert_bitwise(buf.cpu(), OD.embedding_ref(table, ids), "embedding rows (hidden 2048)")
