"""Oracle (test infrastructure): paged KV cache helpers and eager attention on the CPU."""

from __future__ import annotations

import torch


def store_kvcache_ref(key, value, k_cache, v_cache, slot_mapping) -> None:
    """Per token: ``cache.view(-1, H*D)[slot] = src`` unless ``slot == -1``
    (vexact/batch_invariant_ops/kv_cache_context.py:259-276, 294-314). In place."""
    kc = k_cache.view(-1, k_cache.shape[2] * k_cache.shape[3])
    vc = v_cache.view(-1, v_cache.shape[2] * v_cache.shape[3])
    for t in range(key.shape[0]):
        s = int(slot_mapping[t])
        if s == -1:
            continue
        kc[s] = key[t].reshape(-1)
        vc[s] = value[t].reshape(-1)


def make_paged_kv_cache(k_seqs, v_seqs, page_size, perm=None, extra_pages: int = 0):
    """Lay sequences out in pages, ``page_table`` padded with -1
    (tests/batch_invariant_ops/test_triton_attention_varlen.py:26-49). ``perm`` optionally maps the
    consecutive page numbers of that layout to shuffled physical pages."""
    kv_lens = [k.shape[0] for k in k_seqs]
    pages = [(n + page_size - 1) // page_size for n in kv_lens]
    total = sum(pages) + extra_pages
    hk, dk = k_seqs[0].shape[1:]
    dv = v_seqs[0].shape[-1]
    k_cache = torch.zeros(total, page_size, hk, dk, dtype=k_seqs[0].dtype)
    v_cache = torch.zeros(total, page_size, hk, dv, dtype=v_seqs[0].dtype)
    table = torch.full((len(k_seqs), max(pages) if pages else 0), -1, dtype=torch.int32)
    nxt = 0
    for s, n in enumerate(kv_lens):
        for pg in range(pages[s]):
            phys = nxt if perm is None else int(perm[nxt])
            nxt += 1
            lo, hi = pg * page_size, min((pg + 1) * page_size, n)
            table[s, pg] = phys
            k_cache[phys, : hi - lo] = k_seqs[s][lo:hi]
            v_cache[phys, : hi - lo] = v_seqs[s][lo:hi]
    return k_cache, v_cache, table


def gather_paged(cache: torch.Tensor, table_row: torch.Tensor, kv_len: int) -> torch.Tensor:
    """Key ``i`` of a sequence lives at ``cache[table[i // page], i % page]``
    (vexact/batch_invariant_ops/triton_invariant_attention.py:511-526)."""
    page = cache.shape[1]
    idx = torch.arange(kv_len)
    return cache[table_row[idx // page].long(), idx % page]


def eager_attention(q_seq, k_seq, v_seq, softmax_scale, causal=True):
    """fp32 scores and softmax, probabilities cast to the value dtype before ``P @ V``; query ``i``
    sits at absolute position ``kv_len - q_len + i``
    (tests/batch_invariant_ops/test_triton_attention_varlen.py:52-72).
    ``q_seq [Q,Hq,D]``, ``k_seq/v_seq [K,Hkv,D]`` -> ``[Q,Hq,Dv]``."""
    q_t, k_t, v_t = q_seq.transpose(0, 1), k_seq.transpose(0, 1), v_seq.transpose(0, 1)
    groups = q_t.shape[0] // k_t.shape[0]
    if groups != 1:
        k_t = k_t.repeat_interleave(groups, dim=0)
        v_t = v_t.repeat_interleave(groups, dim=0)
    scores = torch.matmul(q_t.float(), k_t.float().transpose(-1, -2)) * softmax_scale
    if causal:
        q_len, kv_len = q_seq.shape[0], k_seq.shape[0]
        q_pos = torch.arange(q_len) + (kv_len - q_len)
        mask = torch.arange(kv_len).unsqueeze(0) <= q_pos.unsqueeze(1)
        scores = scores.masked_fill(~mask.unsqueeze(0), float("-inf"))
    probs = torch.softmax(scores, dim=-1).to(v_seq.dtype)
    if causal:
        probs = torch.where(mask.any(dim=-1)[None, :, None], probs, torch.zeros((), dtype=probs.dtype))
    return torch.matmul(probs.float(), v_t.float()).to(v_seq.dtype).transpose(0, 1)


def paged_attention_ref(q, k_cache, v_cache, cu_seqlens_q, seqused_k, page_table, softmax_scale):
    """Eager attention per sequence after gathering its keys/values from the pages."""
    outs = []
    for s in range(seqused_k.numel()):
        q0, q1 = int(cu_seqlens_q[s]), int(cu_seqlens_q[s + 1])
        n = int(seqused_k[s])
        if q1 <= q0:
            continue
        k = gather_paged(k_cache, page_table[s], n)
        v = gather_paged(v_cache, page_table[s], n)
        outs.append(eager_attention(q[q0:q1], k, v, softmax_scale))
    return torch.cat(outs, dim=0) if outs else q.new_zeros((0, q.shape[1], v_cache.shape[-1]))


def attention_backward_ref(q_seq, k_seq, v_seq, do_seq, softmax_scale):
    """Backward of causal attention for one sequence with the reference's roundings
    (_varlen_attn_bwd_dq_kernel / _varlen_attn_bwd_dkv_kernel, triton_invariant_attention.py:193-430):
    ``P = exp(scale s - lse)``, ``dP = dO V^T``, ``delta = rowsum(O * dO)`` with ``O`` the bf16 forward
    output, ``dS = P (dP - delta) scale``; P and dS are rounded to the input dtype before
    ``dV = P^T dO``, ``dQ = dS K``, ``dK = dS^T Q``; fp32 accumulation, results in the input dtype.
    ``q_seq/do_seq [Q,Hq,D]``, ``k_seq/v_seq [K,Hkv,D]`` -> (dq, dk, dv)."""
    dt = q_seq.dtype
    ql, kl = q_seq.shape[0], k_seq.shape[0]
    g = q_seq.shape[1] // k_seq.shape[1]
    q, do = q_seq.float().transpose(0, 1), do_seq.float().transpose(0, 1)            # [Hq, Q, D]
    k = k_seq.float().transpose(0, 1).repeat_interleave(g, dim=0)                     # [Hq, K, D]
    v = v_seq.float().transpose(0, 1).repeat_interleave(g, dim=0)
    s = torch.matmul(q, k.transpose(-1, -2)) * softmax_scale
    mask = torch.arange(kl).unsqueeze(0) <= (torch.arange(ql) + (kl - ql)).unsqueeze(1)
    s = s.masked_fill(~mask.unsqueeze(0), float("-inf"))
    lse = torch.logsumexp(s, dim=-1, keepdim=True)
    p = torch.where(mask.unsqueeze(0), torch.exp(s - lse), torch.zeros(()))
    p = torch.nan_to_num(p, nan=0.0)                                                  # rows without a visible key
    out = eager_attention(q_seq, k_seq, v_seq, softmax_scale).float().transpose(0, 1)  # bf16 forward output
    delta = (out * do).sum(-1, keepdim=True)
    dp = torch.matmul(do, v.transpose(-1, -2))
    ds = p * (dp - delta) * softmax_scale
    p16, ds16 = p.to(dt).float(), ds.to(dt).float()
    dq = torch.matmul(ds16, k)
    dk = torch.matmul(ds16.transpose(-1, -2), q)
    dv = torch.matmul(p16.transpose(-1, -2), do)
    hkv = k_seq.shape[1]
    dk = dk.reshape(hkv, g, kl, -1).sum(1)                                            # heads of a group, ascending
    dv = dv.reshape(hkv, g, kl, -1).sum(1)
    return dq.transpose(0, 1).to(dt), dk.transpose(0, 1).to(dt), dv.transpose(0, 1).to(dt)
