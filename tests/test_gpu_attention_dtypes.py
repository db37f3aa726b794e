"""GPU parity: attention in fp16 as well as bf16, and on head sizes other than the ones the kernels are built for.

The reference's kernels mask the head dimension to the next power of two and take fp16 or bf16
(vexact/batch_invariant_ops/triton_invariant_attention.py:98-103, 485-490, 645-649, 786-902); its own packed
forward + backward test runs in both dtypes (tests/batch_invariant_ops/test_triton_attention_varlen.py:155-199, restated
first below, with the gradients checked against autograd as well).
"""

import pytest
import torch

from oracle import attention as OA
from tests.util import assert_bitwise

pytestmark = pytest.mark.gpu

from vexact_amd import ops  # noqa: E402
from vexact_amd.batch_invariant_ops import triton_flash_attn_varlen_func as flash_attn_varlen_func  # noqa: E402


def _cu(lens):
    out = [0]
    for n in lens:
        out.append(out[-1] + n)
    return torch.tensor(out, dtype=torch.int32)


def _seqs(lens, heads, dim, seed, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(n, heads, dim, generator=g) * scale).to(dtype) for n in lens]


def _packed_fwd_bwd(q_seqs, k_seqs, v_seqs, do_seqs):
    q = torch.cat(q_seqs).cuda().requires_grad_()
    k = torch.cat(k_seqs).cuda().requires_grad_()
    v = torch.cat(v_seqs).cuda().requires_grad_()
    q_lens, kv_lens = [t.shape[0] for t in q_seqs], [t.shape[0] for t in k_seqs]
    out, _ = flash_attn_varlen_func(q, k, v, cu_seqlens_q=_cu(q_lens).cuda(), cu_seqlens_k=_cu(kv_lens).cuda(),
                                    max_seqlen_q=max(q_lens), max_seqlen_k=max(kv_lens), causal=True)
    out.backward(torch.cat(do_seqs).cuda())
    return out.detach().cpu(), q.grad.cpu(), k.grad.cpu(), v.grad.cpu()


def _autograd_reference(q, k, v, do, scale):
    """fp32 eager causal attention of one sequence and its gradients by autograd."""
    ql, kl = q.shape[0], k.shape[0]
    qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
    g = q.shape[1] // k.shape[1]
    sc = torch.einsum("qhd,khd->hqk", qf, kf.repeat_interleave(g, dim=1)) * scale
    mask = torch.arange(kl)[None, :] <= (torch.arange(ql) + (kl - ql))[:, None]
    sc = sc.masked_fill(~mask[None], float("-inf"))
    ref = torch.einsum("hqk,khd->qhd", torch.softmax(sc, -1), vf.repeat_interleave(g, dim=1))
    ref.backward(do.float())
    return ref.detach(), qf.grad, kf.grad, vf.grad


@pytest.mark.parametrize(("dtype", "atol", "rtol"), [(torch.float16, 2e-2, 2e-2), (torch.bfloat16, 3e-2, 3e-2)])
def test_packed_forward_and_backward_in_both_dtypes(dtype, atol, rtol):
    # the reference's test_triton_flash_attn_varlen_nonpaged_packed_backward: same shapes, seeds' role, tolerances
    print(f"[case] packed forward + backward {dtype}", flush=True)
    q_lens = kv_lens = [65, 129]
    qh, kh, d = 4, 2, 64
    q, k, v = _seqs(q_lens, qh, d, 0, dtype), _seqs(kv_lens, kh, d, 1, dtype), _seqs(kv_lens, kh, d, 2, dtype)
    qg, kg, vg = (torch.cat(t).cuda().requires_grad_() for t in (q, k, v))
    out, _ = flash_attn_varlen_func(qg, kg, vg, _cu(q_lens).cuda(), _cu(kv_lens).cuda(), max_seqlen_q=max(q_lens),
                                    max_seqlen_k=max(kv_lens), softmax_scale=d**-0.5, causal=True)
    assert out.dtype == dtype
    ref = torch.cat([OA.eager_attention(a, b, c, d**-0.5) for a, b, c in zip(q, k, v)])
    torch.testing.assert_close(out.detach().cpu(), ref, atol=atol, rtol=rtol)
    out.square().sum().backward()
    for t in (qg, kg, vg):
        assert t.grad is not None and t.grad.dtype == dtype and bool(torch.isfinite(t.grad).all())
    # beyond the reference's "finite": the gradients of that loss against autograd through fp32 eager attention
    o = 0
    for s, n in enumerate(q_lens):
        want_out, dq, dk, dv = _autograd_reference(q[s], k[s], v[s], 2 * out.detach()[o : o + n].cpu(), d**-0.5)
        for name, got, want in (("dq", qg.grad[o : o + n], dq), ("dk", kg.grad[o : o + n], dk), ("dv", vg.grad[o : o + n], dv)):
            err = (got.float().cpu() - want).abs()
            top = float(want.abs().max())
            assert float(err.max()) <= 2e-2 * top and float(err.mean()) <= 2e-3 * top, (
                f"{name} of sequence {s}: max {float(err.max()):.4g}, mean {float(err.mean()):.4g}, scale {top:.4g}")
        o += n


def _run_paged(q_seqs, k_seqs, v_seqs, page, max_seqlen_q=None, decode_kernel="auto"):
    k_cache, v_cache, table = OA.make_paged_kv_cache(k_seqs, v_seqs, page)
    q_lens = [t.shape[0] for t in q_seqs]
    used = torch.tensor([t.shape[0] for t in k_seqs], dtype=torch.int32)
    mq = max(q_lens) if max_seqlen_q is None else max_seqlen_q
    if decode_kernel != "auto":
        return ops.paged_attention(torch.cat(q_seqs).cuda(), k_cache.cuda(), v_cache.cuda(), _cu(q_lens).cuda(), used.cuda(),
                                   table.cuda(), q_seqs[0].shape[-1] ** -0.5, mq, decode_kernel=decode_kernel)
    out, _ = flash_attn_varlen_func(torch.cat(q_seqs).cuda(), k_cache.cuda(), v_cache.cuda(), cu_seqlens_q=_cu(q_lens).cuda(),
                                    max_seqlen_q=mq, seqused_k=used.cuda(), causal=True, page_table=table.cuda())
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize(("qh", "kh", "dk", "dv"), [
    (8, 2, 96, 96), (4, 2, 80, 80),     # between the built-for sizes
    (4, 4, 40, 24), (6, 2, 160, 128),   # unequal, incl. the 256 / 128 pair
    (4, 2, 200, 136),                   # two sets of output accumulators
    (4, 2, 100, 72), (4, 1, 33, 17),    # not multiples of 8: per-element accesses
    (40, 2, 96, 96),                    # more than 16 query heads per kv head (two query tiles per wavefront)
])
def test_head_sizes_between_the_built_for_ones(dtype, qh, kh, dk, dv):
    print(f"[case] head sizes {dk}/{dv} Hq={qh} Hkv={kh} {dtype}", flush=True)
    page = 16
    q_lens = [70, 1, 33, 1, 5]
    kv_lens = [70, 300, 33, 257, 64]
    q = _seqs(q_lens, qh, dk, 11, dtype, 0.3)
    k = _seqs(kv_lens, kh, dk, 12, dtype, 0.3)
    v = _seqs(kv_lens, kh, dv, 13, dtype, 0.3)
    out = _run_paged(q, k, v, page)
    assert out.dtype == dtype and out.shape == (sum(q_lens), qh, dv)
    ref = torch.cat([OA.eager_attention(a, b, c, dk**-0.5) for a, b, c in zip(q, k, v)])
    torch.testing.assert_close(out.cpu(), ref, atol=3e-3, rtol=3e-3)
    # alone == in the batch, and the last row of a chunk == the decode step of that token (both decode forms)
    o = 0
    for i, (a, b, c) in enumerate(zip(q, k, v)):
        assert_bitwise(_run_paged([a], [b], [c], page), out[o : o + a.shape[0]], f"sequence {i} alone vs in the batch")
        for form in ("split", "fused"):
            dec = _run_paged([a[-1:]], [b], [c], page, max_seqlen_q=1, decode_kernel=form)
            assert_bitwise(dec, out[o + a.shape[0] - 1 : o + a.shape[0]], f"last row of sequence {i} vs its {form} decode step")
        o += a.shape[0]
    # the packed twin gives the paged bits
    packed, _ = flash_attn_varlen_func(torch.cat(q).cuda(), torch.cat(k).cuda(), torch.cat(v).cuda(), cu_seqlens_q=_cu(q_lens).cuda(),
                                       cu_seqlens_k=_cu(kv_lens).cuda(), max_seqlen_q=max(q_lens), max_seqlen_k=max(kv_lens),
                                       causal=True)
    assert_bitwise(packed, out, "packed vs paged")


@pytest.mark.parametrize(("qh", "kh", "d"), [(8, 2, 64), (4, 2, 128), (4, 4, 32)])
def test_padded_kernels_give_the_bits_of_the_exact_size_kernels(qh, kh, d):
    # bf16 at a built-for head size runs the exact-size kernels; the same values behind strides that are not
    # multiples of 8 elements run the padded kernels of the next size (32 -> 64) with per-element accesses.
    # Zeros appended to a score's ascending chain change nothing, so the two must agree in every bit.
    print(f"[case] padded vs exact kernels D={d}", flush=True)
    page = 16
    q_lens, kv_lens = [40, 1, 1], [40, 517, 256]
    q, k, v = _seqs(q_lens, qh, d, 21, torch.bfloat16, 0.3), _seqs(kv_lens, kh, d, 22, torch.bfloat16, 0.3), _seqs(kv_lens, kh, d, 23, torch.bfloat16, 0.3)
    k_cache, v_cache, table = OA.make_paged_kv_cache(k, v, page)
    cu, used = _cu(q_lens).cuda(), torch.tensor(kv_lens, dtype=torch.int32).cuda()

    def odd(t):  # the same values with 4 elements of padding behind every head row: strides % 8 == 4
        buf = torch.zeros(*t.shape[:-1], t.shape[-1] + 4, dtype=t.dtype, device="cuda")
        buf[..., : t.shape[-1]] = t.cuda()
        return buf[..., : t.shape[-1]]

    qa, kc, vc = torch.cat(q).cuda(), k_cache.cuda(), v_cache.cuda()
    exact = ops.paged_attention(qa, kc, vc, cu, used, table.cuda(), d**-0.5, max(q_lens))
    padded = ops.paged_attention(odd(torch.cat(q)), odd(k_cache), odd(v_cache), cu, used, table.cuda(), d**-0.5, max(q_lens))
    assert_bitwise(padded, exact, "general launch")
    qd = torch.cat([t[-1:] for t in q]).cuda()
    cud = torch.arange(len(q_lens) + 1, dtype=torch.int32).cuda()
    for form in ("split", "fused"):
        e = ops.paged_attention(qd, kc, vc, cud, used, table.cuda(), d**-0.5, 1, decode_kernel=form)
        p = ops.paged_attention(odd(qd.cpu()), odd(k_cache), odd(v_cache), cud, used, table.cuda(), d**-0.5, 1, decode_kernel=form)
        assert_bitwise(p, e, f"{form} decode")
    # packed, with the log-sum-exp
    ka, va = torch.cat(k).cuda(), torch.cat(v).cuda()
    e, le = ops.packed_attention(qa, ka, va, cu, _cu(kv_lens).cuda(), d**-0.5, True, max(q_lens), return_lse=True)
    p, lp = ops.packed_attention(odd(torch.cat(q)), odd(torch.cat(k)), odd(torch.cat(v)), cu, _cu(kv_lens).cuda(), d**-0.5, True,
                                 max(q_lens), return_lse=True)
    assert_bitwise(p, e, "packed")
    assert_bitwise(lp, le, "log-sum-exp")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize(("qh", "kh", "dk", "dv", "q_lens", "kv_lens"), [
    (4, 2, 96, 96, [70, 1, 33], [70, 90, 33]),
    (4, 4, 80, 48, [24, 19], [24, 19]),
    (6, 2, 128, 128, [17, 130], [300, 130]),
    (2, 1, 200, 136, [40], [72]),
    (4, 2, 100, 36, [9, 31], [20, 31]),
])
def test_backward_on_other_head_sizes_and_dtypes(dtype, qh, kh, dk, dv, q_lens, kv_lens):
    print(f"[case] attention backward {dtype} Dk={dk} Dv={dv} Hq={qh} Hkv={kh} q={q_lens} kv={kv_lens}", flush=True)
    q, k = _seqs(q_lens, qh, dk, 31, dtype), _seqs(kv_lens, kh, dk, 32, dtype)
    v, do = _seqs(kv_lens, kh, dv, 33, dtype), _seqs(q_lens, qh, dv, 34, dtype)
    out, dq, dk_, dv_ = _packed_fwd_bwd(q, k, v, do)
    scale = dk ** -0.5
    o = ok = 0
    for s, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        _, wq, wk, wv = _autograd_reference(q[s], k[s], v[s], do[s], scale)
        for name, got, want in (("dq", dq[o : o + ql], wq), ("dk", dk_[ok : ok + kl], wk), ("dv", dv_[ok : ok + kl], wv)):
            err = (got.float() - want).abs()
            top = float(want.abs().max())
            assert float(err.max()) <= 2e-2 * top and float(err.mean()) <= 2e-3 * top, (
                f"{name} of sequence {s}: max {float(err.max()):.4g}, mean {float(err.mean()):.4g}, scale {top:.4g}")
        # the restatement with the kernels' roundings of P and dS (tighter)
        odq, odk, odv = OA.attention_backward_ref(q[s], k[s], v[s], do[s], scale)
        for name, got, want in (("dq", dq[o : o + ql], odq), ("dk", dk_[ok : ok + kl], odk), ("dv", dv_[ok : ok + kl], odv)):
            err = (got.float() - want.float()).abs()
            top = float(want.float().abs().max())
            assert float(err.max()) <= 1e-2 * top and float(err.mean()) <= 1e-3 * top, (
                f"{name} of sequence {s} vs the CPU restatement: max {float(err.max()):.4g}, mean {float(err.mean()):.4g}")
        _, dq1, dk1, dv1 = _packed_fwd_bwd(q[s : s + 1], k[s : s + 1], v[s : s + 1], do[s : s + 1])
        assert_bitwise(dq1, dq[o : o + ql], f"dq of sequence {s} alone vs in the batch")
        assert_bitwise(dk1, dk_[ok : ok + kl], f"dk of sequence {s} alone vs in the batch")
        assert_bitwise(dv1, dv_[ok : ok + kl], f"dv of sequence {s} alone vs in the batch")
        o += ql
        ok += kl


def test_backward_register_kernels_agree_with_the_lds_kernels_at_128():
    # bf16 at head size 128 runs the LDS backward kernels; behind unaligned strides the same values run the register
    # kernels built for 128 with per-element accesses. Same formulas, same ascending chains: same bits.
    print("[case] backward: register form vs LDS form at D=128", flush=True)
    q_lens, kv_lens = [130, 5], [200, 5]
    dt = torch.bfloat16
    q, k, v, do = (torch.cat(_seqs(l, h, 128, sd, dt)).cuda() for l, h, sd in ((q_lens, 4, 41), (kv_lens, 2, 42), (kv_lens, 2, 43), (q_lens, 4, 44)))
    cu_q, cu_k = _cu(q_lens).cuda(), _cu(kv_lens).cuda()
    out, lse = ops.packed_attention(q, k, v, cu_q, cu_k, 128**-0.5, True, max(q_lens), return_lse=True)
    want = ops.packed_attention_backward(q, k, v, out, do, lse, cu_q, cu_k, 128**-0.5, max(q_lens), max(kv_lens))

    def odd(t):
        buf = torch.zeros(*t.shape[:-1], t.shape[-1] + 4, dtype=t.dtype, device="cuda")
        buf[..., : t.shape[-1]] = t
        return buf[..., : t.shape[-1]]

    got = ops.packed_attention_backward(odd(q), odd(k), odd(v), odd(out), odd(do), lse, cu_q, cu_k, 128**-0.5, max(q_lens), max(kv_lens))
    for name, a, b in zip(("dq", "dk", "dv"), got, want):
        assert_bitwise(a, b, name)


def test_dtype_and_size_limits_raise():
    q = torch.zeros(2, 4, 64, device="cuda", dtype=torch.float64)
    cu = _cu([2]).cuda()
    with pytest.raises(ValueError, match="bfloat16, float16 or float32"):
        ops.packed_attention(q, q[:, :2], q[:, :2], cu, cu, 0.125, True, 2)
    h = torch.zeros(2, 4, 264, device="cuda", dtype=torch.float16)
    with pytest.raises(ValueError, match="head_dim must be <= 256"):
        ops.packed_attention(h, h[:, :2], h[:, :2], cu, cu, 0.125, True, 2)
    with pytest.raises(ValueError, match="one dtype"):
        ops.packed_attention(h[..., :64], h[:, :2, :64].bfloat16(), h[:, :2, :64], cu, cu, 0.125, True, 2)
