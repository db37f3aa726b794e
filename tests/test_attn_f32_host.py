"""The fp32 attention routines (vexact_amd/csrc/attn_f32.h) compiled for the host and checked against the CPU oracle.

The kernels of the fp32 path are one thread per output row calling these routines, so arithmetic, masks, head mapping,
page lookups and every address are what runs on the GPU. Shapes restate the reference's fp32 tests
(tests/batch_invariant_ops/test_triton_attention_varlen.py:261-300 GQA / q longer than k / head sizes 40 and 96,
:335-395 MLA head sizes 192 / 128) plus paged layouts. Buffers carry NaN guard bands: a read outside a tensor would
poison a result, a write would show in the band.
"""

import ctypes
import os
import subprocess
import tempfile

import numpy as np
import pytest
import torch

from oracle import attention as OA

_HERE = os.path.dirname(os.path.abspath(__file__))
_GUARD = 64


@pytest.fixture(scope="module")
def lib():
    with tempfile.TemporaryDirectory() as d:
        so = os.path.join(d, "attn_f32_harness.so")
        subprocess.run(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-ffp-contract=off", "-o", so,
                        os.path.join(_HERE, "attn_f32_harness.cpp")], check=True)
        yield ctypes.CDLL(so)


def _guarded(t: torch.Tensor):
    """A copy of ``t`` inside a flat fp32 buffer with NaN bands on both sides; returns (buffer, view)."""
    t = t.contiguous()
    buf = torch.full((t.numel() + 2 * _GUARD,), float("nan"), dtype=t.dtype)
    view = buf[_GUARD : _GUARD + t.numel()].view(t.shape)
    view.copy_(t)
    return buf, view


def _bands_intact(buf) -> bool:
    return bool(torch.isnan(buf[:_GUARD]).all() and torch.isnan(buf[-_GUARD:]).all())


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _cu(lens):
    return torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)


def _seqs(lens, heads, dim, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(n, heads, dim, generator=g) for n in lens]


def _forward(lib, q, k, v, cu_q, *, cu_k=None, seqused=None, table=None, page=0, causal=True, scale=None, want_lse=True):
    T, Hq, dk = q.shape
    Hkv, dv = k.shape[-2], v.shape[-1]
    packed = table is None
    qb, qv = _guarded(q)
    kb, kv_ = _guarded(k)
    vb, vv = _guarded(v)
    ob, ov = _guarded(torch.full((T, Hq, dv), 7.0))
    lb, lv = _guarded(torch.full((T, Hq), 7.0))
    B = cu_q.numel() - 1
    max_kv = 0 if packed else table.shape[1] * page
    ints = (ctypes.c_int * 10)(Hq, Hkv, B, dk, dv, int(causal), int(packed), page, max_kv, T)
    if packed:
        st = (qv.stride(0), qv.stride(1), 0, kv_.stride(0), kv_.stride(1), 0, vv.stride(0), vv.stride(1), ov.stride(0), ov.stride(1), 0)
    else:
        st = (qv.stride(0), qv.stride(1), kv_.stride(0), kv_.stride(1), kv_.stride(2), vv.stride(0), vv.stride(1), vv.stride(2),
              ov.stride(0), ov.stride(1), table.stride(0))
    lib.f32_forward(_ptr(qv), _ptr(kv_), _ptr(vv), _ptr(ov), _ptr(lv) if want_lse else None, _ptr(cu_q), _ptr(seqused),
                    _ptr(cu_k), _ptr(table), ints, (ctypes.c_int64 * 11)(*st),
                    ctypes.c_float(dk ** -0.5 if scale is None else scale))
    assert all(_bands_intact(b) for b in (qb, kb, vb, ob, lb)), "a guard band was written"
    return ov.clone(), lv.clone()


def _backward(lib, q, k, v, o, do, lse, cu_q, cu_k, scale):
    T, Hq, dk = q.shape
    Tk, Hkv, dv = v.shape
    bufs = [_guarded(t) for t in (q, k, v, o, do, lse, torch.zeros(T, Hq), torch.full_like(q, 7.0), torch.full_like(k, 7.0),
                                  torch.full_like(v, 7.0))]
    (qv, kv_, vv, ov, dov, lv, delta, dq, dk_, dv_) = [b[1] for b in bufs]
    ints = (ctypes.c_int * 7)(Hq, Hkv, cu_q.numel() - 1, dk, dv, T, Tk)
    st = [s for t in (qv, kv_, vv, ov, dov, dq, dk_, dv_) for s in (t.stride(0), t.stride(1))]
    lib.f32_backward(_ptr(qv), _ptr(kv_), _ptr(vv), _ptr(ov), _ptr(dov), _ptr(lv), _ptr(delta), _ptr(dq), _ptr(dk_), _ptr(dv_),
                     _ptr(cu_q), _ptr(cu_k), ints, (ctypes.c_int64 * 16)(*st), ctypes.c_float(scale))
    assert all(_bands_intact(b[0]) for b in bufs), "a guard band was written"
    return dq.clone(), dk_.clone(), dv_.clone()


CASES = [  # q_lens, kv_lens, q heads, kv heads, dk, dv
    ([17, 33, 65], [17, 33, 65], 4, 2, 64, 64),
    ([1, 7, 19], [65, 71, 83], 4, 2, 64, 64),
    ([5, 9], [2, 4], 4, 2, 32, 32),          # queries that see no key at all
    ([9, 23], [41, 57], 6, 3, 40, 40),
    ([9, 23], [41, 57], 6, 3, 96, 96),
    ([3, 17], [33, 65], 16, 16, 192, 128),   # MLA
    ([4, 0, 6], [4, 0, 9], 2, 1, 8, 8),      # an empty sequence in the middle
]


@pytest.mark.parametrize("q_lens,kv_lens,qh,kh,dk,dv", CASES)
def test_packed_forward_and_backward_match_eager_autograd(lib, q_lens, kv_lens, qh, kh, dk, dv):
    q_seqs, k_seqs, v_seqs = _seqs(q_lens, qh, dk, 1), _seqs(kv_lens, kh, dk, 2), _seqs(kv_lens, kh, dv, 3)
    do_seqs = _seqs(q_lens, qh, dv, 4)
    q, k, v, do = (torch.cat(s) for s in (q_seqs, k_seqs, v_seqs, do_seqs))
    cu_q, cu_k = _cu(q_lens), _cu(kv_lens)
    scale = dk ** -0.5
    out, lse = _forward(lib, q, k, v, cu_q, cu_k=cu_k)
    dq, dk_, dv_ = _backward(lib, q, k, v, out, do, lse, cu_q, cu_k, scale)
    oq = ok = 0
    for s, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        if ql == 0:
            continue
        qf, kf, vf = (t.clone().double().requires_grad_() for t in (q_seqs[s], k_seqs[s], v_seqs[s]))
        ref = OA.eager_attention(qf, kf, vf, scale)
        ref.backward(do_seqs[s].double())
        torch.testing.assert_close(out[oq : oq + ql].double(), ref.detach(), atol=2e-6, rtol=1e-5)
        torch.testing.assert_close(dq[oq : oq + ql].double(), qf.grad, atol=1e-5, rtol=1e-4)
        torch.testing.assert_close(dk_[ok : ok + kl].double(), kf.grad, atol=1e-5, rtol=1e-4)
        torch.testing.assert_close(dv_[ok : ok + kl].double(), vf.grad, atol=1e-5, rtol=1e-4)
        # log-sum-exp of the visible scores; +inf for a row that sees nothing
        pos = torch.arange(ql) + (kl - ql)
        sc = torch.einsum("qhd,khd->qhk", qf.detach(), kf.detach().repeat_interleave(qh // kh, dim=1)) * scale
        sc = sc.masked_fill(~(torch.arange(kl)[None, :] <= pos[:, None])[:, None, :], float("-inf"))
        want = torch.logsumexp(sc, -1)
        dead = pos < 0
        assert torch.isinf(lse[oq : oq + ql][dead]).all() and (out[oq : oq + ql][dead] == 0).all()
        torch.testing.assert_close(lse[oq : oq + ql][~dead].double(), want[~dead], atol=1e-5, rtol=1e-5)
        # the sequence alone: same bits
        o1, l1 = _forward(lib, q_seqs[s], k_seqs[s], v_seqs[s], _cu([ql]), cu_k=_cu([kl]))
        g1 = _backward(lib, q_seqs[s], k_seqs[s], v_seqs[s], o1, do_seqs[s], l1, _cu([ql]), _cu([kl]), scale)
        assert torch.equal(o1, out[oq : oq + ql])
        assert torch.equal(g1[0], dq[oq : oq + ql]) and torch.equal(g1[1], dk_[ok : ok + kl]) and torch.equal(g1[2], dv_[ok : ok + kl])
        oq += ql
        ok += kl


def test_non_causal_packed_forward(lib):
    q, k, v = _seqs([5], 4, 16, 1)[0], _seqs([9], 2, 16, 2)[0], _seqs([9], 2, 16, 3)[0]
    out, _ = _forward(lib, q, k, v, _cu([5]), cu_k=_cu([9]), causal=False)
    torch.testing.assert_close(out.double(), OA.eager_attention(q.double(), k.double(), v.double(), 0.25, causal=False),
                               atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("page", [16, 5])
def test_paged_layout_gives_the_bits_of_the_packed_layout_and_decode_those_of_prefill(lib, page):
    kv_lens, qh, kh, d = [17, 33, 64, 1], 4, 2, 32
    q_seqs, k_seqs, v_seqs = _seqs(kv_lens, qh, d, 5), _seqs(kv_lens, kh, d, 6), _seqs(kv_lens, kh, d, 7)
    perm = torch.randperm(sum((n + page - 1) // page for n in kv_lens) + 3, generator=torch.Generator().manual_seed(8))
    k_cache, v_cache, table = OA.make_paged_kv_cache(k_seqs, v_seqs, page, perm=perm, extra_pages=3)
    used = torch.tensor(kv_lens, dtype=torch.int32)
    packed, _ = _forward(lib, torch.cat(q_seqs), torch.cat(k_seqs), torch.cat(v_seqs), _cu(kv_lens), cu_k=_cu(kv_lens))
    paged, _ = _forward(lib, torch.cat(q_seqs), k_cache, v_cache, _cu(kv_lens), seqused=used, table=table, page=page, want_lse=False)
    assert torch.equal(paged, packed)
    ref = OA.paged_attention_ref(torch.cat(q_seqs).double(), k_cache.double(), v_cache.double(), _cu(kv_lens), used, table, d ** -0.5)
    torch.testing.assert_close(paged.double(), ref, atol=2e-6, rtol=1e-5)
    # decode: the last token of every sequence alone, over the same pages
    last = torch.stack([s[-1] for s in q_seqs])
    dec, _ = _forward(lib, last, k_cache, v_cache, _cu([1] * len(kv_lens)), seqused=used, table=table, page=page, want_lse=False)
    ends = np.cumsum(kv_lens) - 1
    assert torch.equal(dec, paged[ends])
    # a sequence without keys is left alone; a length beyond the table is clamped to what the table addresses
    used0 = used.clone()
    used0[1] = 0
    out0, _ = _forward(lib, torch.cat(q_seqs), k_cache, v_cache, _cu(kv_lens), seqused=used0, table=table, page=page, want_lse=False)
    assert (out0[17 : 17 + 33] == 7.0).all() and torch.equal(out0[:17], paged[:17])


def test_addresses_under_address_and_ub_sanitizers():
    # random packed and paged batches (ragged and empty sequences, odd head sizes and page sizes, a kv length beyond what
    # the block table addresses) with exactly sized heap buffers, compiled with -fsanitize=address,undefined
    with tempfile.TemporaryDirectory() as d:
        exe = os.path.join(d, "attn_f32_sanitized")
        subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                        "-static-libasan", "-ffp-contract=off", "-o", exe, os.path.join(_HERE, "attn_f32_sanitized.cpp")], check=True)
        run = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "sanitized run ok" in run.stdout
