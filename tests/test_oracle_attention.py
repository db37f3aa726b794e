"""Pins the attention / KV-cache oracle: fp64 brute force, closed-form special cases, round trips."""

import math

import torch

from oracle import attention as OA


def _seqs(lens, heads, dim, seed, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(n, heads, dim, generator=g) * scale).to(dtype) for n in lens]


def _brute(q, k, v, scale, causal=True):
    Q, Hq, D = q.shape
    K, Hkv, Dv = v.shape
    out = torch.zeros(Q, Hq, Dv, dtype=torch.float64)
    for i in range(Q):
        pos = K - Q + i if causal else K - 1
        for h in range(Hq):
            kh = h // (Hq // Hkv)
            s = [sum(float(q[i, h, d]) * float(k[j, kh, d]) for d in range(D)) * scale for j in range(pos + 1)]
            m = max(s)
            e = [math.exp(x - m) for x in s]
            z = sum(e)
            for j in range(pos + 1):
                out[i, h] += (e[j] / z) * v[j, kh].double()
    return out


def test_eager_attention_matches_fp64_brute_force():
    q, k, v = _seqs([3], 4, 8, 1)[0], _seqs([6], 2, 8, 2)[0], _seqs([6], 2, 8, 3)[0]
    got = OA.eager_attention(q, k, v, 8 ** -0.5)
    want = _brute(q, k, v, 8 ** -0.5)
    assert (got.double() - want).abs().max() < 2e-2  # bf16 probabilities and output
    # fp32 inputs: only float rounding remains; wrong masks / positions / head mapping would show
    qf, kf, vf = q.float(), k.float(), v.float()
    assert (OA.eager_attention(qf, kf, vf, 8 ** -0.5).double() - _brute(qf, kf, vf, 8 ** -0.5)).abs().max() < 1e-5
    nc = OA.eager_attention(qf, kf, vf, 8 ** -0.5, causal=False)
    assert (nc.double() - _brute(qf, kf, vf, 8 ** -0.5, causal=False)).abs().max() < 1e-5


def test_special_cases():
    # one key: the output is that key's value
    q, k, v = _seqs([1], 4, 16, 4)[0], _seqs([1], 2, 16, 5)[0], _seqs([1], 2, 16, 6)[0]
    assert torch.equal(OA.eager_attention(q, k, v, 0.25), v.repeat_interleave(2, dim=1))
    # identical keys: uniform probabilities, output = running mean of the visible values
    kk = _seqs([1], 1, 8, 7, dtype=torch.float32)[0].repeat(5, 1, 1)
    vv = _seqs([5], 1, 8, 8, dtype=torch.float32)[0]
    qq = _seqs([5], 1, 8, 9, dtype=torch.float32)[0]
    got = OA.eager_attention(qq, kk, vv, 1.0)
    for i in range(5):
        torch.testing.assert_close(got[i, 0], vv[: i + 1, 0].mean(0), atol=1e-6, rtol=1e-5)


def test_paged_layout_round_trip_and_store():
    ks, vs = _seqs([17, 33, 5], 2, 8, 10), _seqs([17, 33, 5], 2, 8, 11)
    perm = torch.randperm(12, generator=torch.Generator().manual_seed(12))
    kc, vc, table = OA.make_paged_kv_cache(ks, vs, 8, perm=perm, extra_pages=2)
    assert table.shape == (3, 5) and table[0, 3] == -1 and table[2, 1] == -1
    assert sorted(table[table >= 0].tolist()) == sorted(perm[:9].tolist())
    for s, n in enumerate([17, 33, 5]):
        assert torch.equal(OA.gather_paged(kc, table[s], n), ks[s])
        assert torch.equal(OA.gather_paged(vc, table[s], n), vs[s])
    # store: loop restatement == vectorised indexing; -1 rows untouched
    key, val = _seqs([9], 2, 8, 13)[0], _seqs([9], 2, 8, 14)[0]
    slots = torch.tensor([5, 0, -1, 40, 41, 7, -1, 85, 12], dtype=torch.int32)
    kc2, vc2 = kc.clone(), vc.clone()
    OA.store_kvcache_ref(key, val, kc2, vc2, slots)
    want = kc.clone().view(-1, 16)
    keep = slots >= 0
    want[slots[keep].long()] = key[keep].reshape(-1, 16)
    assert torch.equal(kc2.view(-1, 16), want)
    untouched = torch.ones(88, dtype=torch.bool)
    untouched[slots[keep].long()] = False
    assert torch.equal(vc2.view(-1, 16)[untouched], vc.view(-1, 16)[untouched])


def test_paged_attention_ref_equals_eager_on_gathered_keys():
    qs, ks, vs = _seqs([1, 4], 4, 16, 15), _seqs([20, 9], 2, 16, 16), _seqs([20, 9], 2, 16, 17)
    kc, vc, table = OA.make_paged_kv_cache(ks, vs, 4)
    cu = torch.tensor([0, 1, 5], dtype=torch.int32)
    used = torch.tensor([20, 9], dtype=torch.int32)
    got = OA.paged_attention_ref(torch.cat(qs), kc, vc, cu, used, table, 0.25)
    want = torch.cat([OA.eager_attention(a, b, c, 0.25) for a, b, c in zip(qs, ks, vs)])
    assert torch.equal(got, want)


def test_attention_backward_restatement_matches_autograd():
    # the reference's backward formulas (with bf16 P and dS) against autograd through the fp32 eager
    # attention; a single visible key makes P = 1 exactly: dV = dO, dQ = dK = 0
    g = torch.Generator().manual_seed(3)
    for (ql, kl, hq, hkv, d) in ((9, 9, 4, 2, 32), (5, 23, 6, 2, 64), (1, 40, 2, 2, 32)):
        q = torch.randn(ql, hq, d, generator=g).to(torch.bfloat16)
        k = torch.randn(kl, hkv, d, generator=g).to(torch.bfloat16)
        v = torch.randn(kl, hkv, d, generator=g).to(torch.bfloat16)
        do = torch.randn(ql, hq, d, generator=g).to(torch.bfloat16)
        dq, dk, dv = OA.attention_backward_ref(q, k, v, do, d ** -0.5)
        qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
        grp = hq // hkv
        s = torch.einsum("qhd,khd->hqk", qf, kf.repeat_interleave(grp, dim=1)) * d ** -0.5
        mask = torch.arange(kl)[None, :] <= (torch.arange(ql) + (kl - ql))[:, None]
        o = torch.einsum("hqk,khd->qhd", torch.softmax(s.masked_fill(~mask[None], float("-inf")), -1), vf.repeat_interleave(grp, dim=1))
        o.backward(do.float())
        for name, got, want in (("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad)):
            err = (got.float() - want).abs().max()
            assert float(err) <= 2e-2 * float(want.abs().max()), (name, ql, kl, float(err))
    q = torch.randn(1, 2, 32, generator=g).to(torch.bfloat16)
    k = torch.randn(1, 2, 32, generator=g).to(torch.bfloat16)
    v = torch.randn(1, 2, 32, generator=g).to(torch.bfloat16)
    do = torch.randn(1, 2, 32, generator=g).to(torch.bfloat16)
    dq, dk, dv = OA.attention_backward_ref(q, k, v, do, 0.3)
    assert torch.equal(dv, do) and float(dq.abs().max()) < 1e-2 and float(dk.abs().max()) < 1e-2
