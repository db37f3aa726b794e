"""Pins the MoE oracle: brute-force routing, closed-form special cases of the expert MLP."""

import numpy as np
import torch
import torch.nn.functional as F

from oracle import moe as OM


def _w(E, I, H, seed, scale=0.1):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: (torch.randn(*s, generator=g) * scale).to(torch.bfloat16)  # noqa: E731
    return mk(E, I, H), mk(E, I, H), mk(E, H, I)


def test_router_ref_against_python_topk():
    g = torch.Generator().manual_seed(1)
    logits = torch.randn(9, 12, generator=g)
    logits[2, 4] = logits[2, 7]  # tie: lower index first
    w, idx = OM.router_ref(logits, 3, renorm=True, out_dtype=torch.float32)
    probs = torch.softmax(logits.double(), -1)
    for t in range(9):
        order = sorted(range(12), key=lambda e: (-float(torch.softmax(logits[t], -1)[e]), e))[:3]
        assert idx[t].tolist() == order
        want = probs[t, order] / probs[t, order].sum()
        torch.testing.assert_close(w[t].double(), want, atol=1e-6, rtol=1e-5)
    assert idx[2].tolist().index(4) < idx[2].tolist().index(7) if (4 in idx[2].tolist() and 7 in idx[2].tolist()) else True
    w2, _ = OM.router_ref(logits, 3, renorm=False, out_dtype=torch.float32)
    torch.testing.assert_close(w2.sum(-1).double(), probs.gather(-1, idx).sum(-1), atol=1e-6, rtol=1e-5)
    wf = OM.router_weights_for(logits, idx, renorm=True, out_dtype=torch.float32)
    assert torch.equal(wf, w)


def test_routing_integers_against_counting():
    g = torch.Generator().manual_seed(2)
    sel = torch.randint(0, 5, (11, 3), generator=g)
    r = OM.routing_integers_ref(sel, 5)
    flat = sel.reshape(-1).tolist()
    assert r["splits"].tolist() == [flat.count(e) for e in range(5)]
    assert r["cu"].tolist() == [sum(flat.count(x) for x in range(e)) for e in range(6)]
    for f, e in enumerate(flat):
        rank = sum(1 for x in flat if x < e) + sum(1 for x in flat[:f] if x == e)
        assert r["scatter_index"].reshape(-1)[f] == rank
        assert r["sorted_flat"][rank] == f and r["sorted_token"][rank] == f // 3
    # the reference's own formulation: argsort(stable).argsort()
    twice = sel.flatten().argsort(stable=True).argsort().int().view(sel.shape)
    assert np.array_equal(twice.numpy(), r["scatter_index"])
    tg, t0, tr = OM.tile_table_ref(r["splits"], 4)
    assert int(tr.sum()) == 33 and all(x <= 4 for x in tr)
    assert all(r["cu"][g_] <= a < r["cu"][g_ + 1] for g_, a in zip(tg, t0))


def test_fused_moe_ref_special_cases():
    E, I, H, T = 4, 16, 24, 7
    gate, up, down = _w(E, I, H, 3)
    x = (torch.randn(T, H, generator=torch.Generator().manual_seed(4))).to(torch.bfloat16)
    bf = lambda t: t.to(torch.bfloat16)  # noqa: E731
    # k = 1, weight 1: a plain SwiGLU MLP of the chosen expert with bf16 roundings
    sel = torch.tensor([[t % E] for t in range(T)])
    w = torch.ones(T, 1, dtype=torch.bfloat16)
    got = OM.fused_moe_ref(x, w, sel, gate, up, down)
    for t in range(T):
        e = t % E
        g_ = bf(x[t].float() @ gate[e].float().t())
        u_ = bf(x[t].float() @ up[e].float().t())
        h_ = bf(bf(F.silu(g_.float())).float() * u_.float())
        o_ = bf(h_.float() @ down[e].float().t())
        assert torch.equal(got[t], o_)
    # every token on one expert twice with weights a, b: slots are summed in fp32, slot order
    sel2 = torch.full((T, 2), 2)
    w2 = torch.tensor([[0.75, 0.25]] * T, dtype=torch.bfloat16)
    got2 = OM.fused_moe_ref(x, w2, sel2, gate, up, down)
    g_ = bf(x.float() @ gate[2].float().t())
    u_ = bf(x.float() @ up[2].float().t())
    h_ = bf(bf(F.silu(g_.float())).float() * u_.float())
    o0 = bf(bf(h_.float() * 0.75).float() @ down[2].float().t())
    o1 = bf(bf(h_.float() * 0.25).float() @ down[2].float().t())
    assert torch.equal(got2, bf(o0.float() + o1.float()))
    # fp64 restatement without intermediate rounding is close; the HF-eager order too
    sel3 = torch.tensor([[0, 3], [1, 2], [3, 0], [2, 2], [1, 0], [0, 1], [3, 2]])
    w3 = torch.softmax(torch.randn(T, 2, generator=torch.Generator().manual_seed(5)), -1).to(torch.bfloat16)
    got3 = OM.fused_moe_ref(x, w3, sel3, gate, up, down).double()
    want = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for i in range(2):
            e = int(sel3[t, i])
            hh = F.silu(x[t].double() @ gate[e].double().t()) * (x[t].double() @ up[e].double().t())
            want[t] += float(w3[t, i]) * (hh @ down[e].double().t())
    assert (got3 - want).abs().max() <= 3e-2 * want.abs().max()
    hf = OM.hf_eager_moe_ref(x, w3, sel3, gate, up, down).double()
    assert (hf - want).abs().max() <= 3e-2 * want.abs().max()


def test_moe_backward_restatement_matches_autograd():
    # the reference's backward formulas (bf16 intermediates) against autograd through an fp32 restatement
    T, H, I, E, k = 24, 32, 16, 4, 2
    g = torch.Generator().manual_seed(2)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    gw, uw = ((torch.randn(E, I, H, generator=g) * 0.2).to(torch.bfloat16) for _ in range(2))
    dw = (torch.randn(E, H, I, generator=g) * 0.2).to(torch.bfloat16)
    w, sel = torch.topk(torch.softmax(torch.randn(T, E, generator=g), -1), k)
    w = (w / w.sum(-1, keepdim=True)).to(torch.bfloat16)
    dy = torch.randn(T, H, generator=g).to(torch.bfloat16)
    got = OM.fused_moe_backward_ref(x, w, sel, gw, uw, dw, dy)
    leaves = [t.float().requires_grad_() for t in (w, x, gw, uw, dw)]
    rw, rx, rg, ru, rd = leaves
    ref = torch.zeros(T, H)
    for i in range(k):
        e = sel[:, i]
        h = torch.nn.functional.silu(torch.einsum("th,tih->ti", rx, rg[e])) * torch.einsum("th,tih->ti", rx, ru[e])
        ref = ref + rw[:, i : i + 1] * torch.einsum("ti,thi->th", h, rd[e])
    ref.backward(dy.float())
    for name, a, b in zip(("routing weights", "hidden", "gate", "up", "down"), got, leaves):
        err = (a.float() - b.grad).abs()
        assert float(err.max()) <= 3e-2 * float(b.grad.abs().max()), (name, float(err.max()), float(b.grad.abs().max()))
