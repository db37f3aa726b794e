"""GPU parity: attention on fp32 tensors, and queries that see no key.

The reference's attention takes fp32 as well (vexact/batch_invariant_ops/triton_invariant_attention.py:108-113) and its
own backward tests run in it: tests/batch_invariant_ops/test_triton_attention_varlen.py:261-273 (GQA), :275-287 (more
queries than keys), :290-302 (head sizes 40 and 96), :335-395 (head sizes 192 / 128), restated below through the same
public function, with the reference's tolerances as the bar and the measured distance printed (true fp32 products here,
TF32 there). The routines behind the kernels are also checked on the host (tests/test_attn_f32_host.py).
"""

import pytest
import torch

from oracle import attention as OA
from tests.util import assert_bitwise

pytestmark = pytest.mark.gpu

from vexact_amd.batch_invariant_ops import triton_flash_attn_varlen_func as flash_attn_varlen_func  # noqa: E402


def _cu(lens):
    out = [0]
    for n in lens:
        out.append(out[-1] + n)
    return torch.tensor(out, dtype=torch.int32)


def _seqs(lens, heads, dim, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(n, heads, dim, generator=g).to(dtype) for n in lens]


def _packed_fwd_bwd(q_seqs, k_seqs, v_seqs, do_seqs):
    q = torch.cat(q_seqs).cuda().requires_grad_()
    k = torch.cat(k_seqs).cuda().requires_grad_()
    v = torch.cat(v_seqs).cuda().requires_grad_()
    q_lens, kv_lens = [t.shape[0] for t in q_seqs], [t.shape[0] for t in k_seqs]
    out, _ = flash_attn_varlen_func(q, k, v, cu_seqlens_q=_cu(q_lens).cuda(), cu_seqlens_k=_cu(kv_lens).cuda(),
                                    max_seqlen_q=max(q_lens), max_seqlen_k=max(kv_lens), softmax_scale=q.shape[-1] ** -0.5,
                                    causal=True)
    out.backward(torch.cat(do_seqs).cuda())
    return out.detach().cpu(), q.grad.cpu(), k.grad.cpu(), v.grad.cpu()


def _check_against_eager(q_lens, kv_lens, qh, kh, dk, dv, dtype, atol, rtol, seed):
    print(f"[case] packed forward + backward {dtype} Hq={qh} Hkv={kh} D={dk}/{dv} q={q_lens} kv={kv_lens}", flush=True)
    q_seqs, k_seqs, v_seqs = _seqs(q_lens, qh, dk, seed, dtype), _seqs(kv_lens, kh, dk, seed + 1, dtype), _seqs(kv_lens, kh, dv, seed + 2, dtype)
    do_seqs = _seqs(q_lens, qh, dv, seed + 3, dtype)
    out, dq, dk_, dv_ = _packed_fwd_bwd(q_seqs, k_seqs, v_seqs, do_seqs)
    assert out.dtype == dtype and dq.dtype == dtype
    oq = ok = 0
    worst = 0.0
    for s, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        qf, kf, vf = (t.clone().requires_grad_() for t in (q_seqs[s], k_seqs[s], v_seqs[s]))
        ref = OA.eager_attention(qf, kf, vf, dk ** -0.5)  # the reference test's _eager_attention
        ref.backward(do_seqs[s])
        for name, got, want in (("out", out[oq : oq + ql], ref.detach()), ("dq", dq[oq : oq + ql], qf.grad),
                                ("dk", dk_[ok : ok + kl], kf.grad), ("dv", dv_[ok : ok + kl], vf.grad)):
            worst = max(worst, float((got.float() - want.float()).abs().max()))
            torch.testing.assert_close(got, want, atol=atol, rtol=rtol, msg=lambda m: f"{name} of sequence {s}: {m}")
        # the sequence alone gives the same bits
        o1, dq1, dk1, dv1 = _packed_fwd_bwd(q_seqs[s : s + 1], k_seqs[s : s + 1], v_seqs[s : s + 1], do_seqs[s : s + 1])
        assert_bitwise(o1, out[oq : oq + ql], f"out of sequence {s} alone vs in the batch")
        assert_bitwise(dq1, dq[oq : oq + ql], f"dq of sequence {s} alone vs in the batch")
        assert_bitwise(dk1, dk_[ok : ok + kl], f"dk of sequence {s} alone vs in the batch")
        assert_bitwise(dv1, dv_[ok : ok + kl], f"dv of sequence {s} alone vs in the batch")
        oq += ql
        ok += kl
    print(f"[fp32] largest |difference| from the eager reference {worst:.3e} (bound {atol:g})", flush=True)


@pytest.mark.parametrize(("q_lens", "kv_lens"), [([17, 33, 65], [17, 33, 65]), ([1, 7, 19], [65, 71, 83])])
def test_fp32_gqa_backward_matches_eager(q_lens, kv_lens):
    _check_against_eager(q_lens, kv_lens, 4, 2, 64, 64, torch.float32, 5e-3, 5e-3, seed=101)


def test_fp32_more_queries_than_keys_matches_eager():
    # the first q_len - kv_len rows see no key: output and gradient 0, as the eager reference defines them
    _check_against_eager([5, 9], [2, 4], 4, 2, 32, 32, torch.float32, 2e-3, 2e-3, seed=303)


@pytest.mark.parametrize("head_dim", [40, 96])
def test_fp32_arbitrary_head_dim_backward_matches_eager(head_dim):
    _check_against_eager([9, 23], [41, 57], 6, 3, head_dim, head_dim, torch.float32, 7e-3, 7e-3, seed=202)


def test_fp32_mla_head_dims_backward_matches_eager():
    _check_against_eager([3, 17], [33, 65], 16, 16, 192, 128, torch.float32, 5e-3, 5e-3, seed=404)


@pytest.mark.parametrize(("dtype", "atol"), [(torch.bfloat16, 3e-2), (torch.float16, 2e-2)])
def test_more_queries_than_keys_in_the_16_bit_types(dtype, atol):
    _check_against_eager([5, 9], [2, 4], 4, 2, 32, 32, dtype, atol, atol, seed=305)


def test_fp32_paged_correctness_batch_invariance_and_prefill_decode_alignment():
    qh, kh, d, page = 4, 2, 32, 16
    kv_lens = [17, 33, 64, 5]
    q_seqs, k_seqs, v_seqs = _seqs(kv_lens, qh, d, 11), _seqs(kv_lens, kh, d, 12), _seqs(kv_lens, kh, d, 13)
    k_cache, v_cache, table = OA.make_paged_kv_cache(k_seqs, v_seqs, page)
    used = torch.tensor(kv_lens, dtype=torch.int32)

    def run(qs, rows):
        lens = [t.shape[0] for t in qs]
        return flash_attn_varlen_func(torch.cat(qs).cuda(), k_cache.cuda(), v_cache.cuda(), cu_seqlens_q=_cu(lens).cuda(),
                                      max_seqlen_q=max(lens), seqused_k=used[rows].cuda(), page_table=table[rows].cuda(),
                                      softmax_scale=d ** -0.5, causal=True)[0].cpu()

    everything = list(range(len(kv_lens)))
    out = run(q_seqs, everything)
    ref = OA.paged_attention_ref(torch.cat(q_seqs), k_cache, v_cache, _cu(kv_lens), used, table, d ** -0.5)
    torch.testing.assert_close(out, ref, atol=2e-3, rtol=2e-3)
    print(f"[fp32] paged: largest |difference| from the eager reference {float((out - ref).abs().max()):.3e}", flush=True)
    o = 0
    for s, n in enumerate(kv_lens):
        assert_bitwise(run(q_seqs[s : s + 1], [s]), out[o : o + n], f"sequence {s} alone vs in the batch")
        o += n
    # decode: the last token of every sequence over the same pages == the last row of its prefill
    dec = run([t[-1:] for t in q_seqs], everything)
    ends = torch.tensor(kv_lens).cumsum(0) - 1
    assert_bitwise(dec, out[ends], "decode step vs last prefill row")
    # packed layout of the same sequences
    packed, _ = flash_attn_varlen_func(torch.cat(q_seqs).cuda(), torch.cat(k_seqs).cuda(), torch.cat(v_seqs).cuda(),
                                       cu_seqlens_q=_cu(kv_lens).cuda(), cu_seqlens_k=_cu(kv_lens).cuda(), max_seqlen_q=max(kv_lens),
                                       max_seqlen_k=max(kv_lens), softmax_scale=d ** -0.5, causal=True)
    assert_bitwise(packed.cpu(), out, "packed vs paged")
