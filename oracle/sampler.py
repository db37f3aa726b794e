"""CPU restatements for the token sampler. TEST INFRASTRUCTURE ONLY.

Two layers:

* ``apply_top_k_top_p_ref`` / ``race_ref`` restate the reference formulas
  (vexact/inferencer/sampler.py:147-189 sort + softmax + cumsum masks, :115-145 ``probs / Exp(1)``
  argmax) in numpy, with the sort made stable and the softmax / cumsum in float64.
* ``sample_tokens_ref`` restates, operation for operation in float32 / integer numpy, the
  specification the HIP sampler implements (integer-mass top-p, Philox4x32-10 noise keyed by
  (seed, position, token), polynomial exp / log), so the kernel can be checked bit for bit.

The second is pinned against the first (same kept set on tie-free rows, same token when both are
fed the same exponential variates), against Philox's published known-answer vectors, and against
``numpy.exp`` / ``numpy.log`` for the two polynomials. The reference's seeded path calls vLLM's Triton
Gumbel kernel, which is not in the reference tree: bit parity with that noise stream is unpinned.
"""

from __future__ import annotations

import numpy as np

F = np.float32
CUTOFF = F(-32.0)


# ---------------------------------------------------------------------------------------------
# the reference's formulas
# ---------------------------------------------------------------------------------------------
def apply_top_k_top_p_ref(logits: np.ndarray, k, p) -> np.ndarray:
    """sampler.py:147-189 for one row: ascending (stable) sort, mask below the k-th largest value,
    softmax, cumulative sum, mask while ``cumsum <= 1 - p``, never the last; returns the kept mask."""
    x = logits.astype(np.float64)
    order = np.argsort(x, kind="stable")
    xs = x[order].copy()
    n = xs.size
    if k is not None and 0 < k < n:
        xs[xs < xs[n - k]] = -np.inf
    if p is not None:
        e = np.exp(xs - xs.max())
        cum = np.cumsum(e / e.sum())
        m = cum <= float(F(1.0) - F(p))  # 1 - p is formed in float32 by the reference
        m[-1] = False
        xs[m] = -np.inf
    keep = np.zeros(n, dtype=bool)
    keep[order] = np.isfinite(xs)
    return keep


def race_ref(logits: np.ndarray, keep: np.ndarray, expo: np.ndarray) -> int:
    """sampler.py:143-145: ``argmax(softmax(masked logits) / q)`` with q ~ Exp(1) given in ``expo``."""
    x = np.where(keep, logits.astype(np.float64), -np.inf)
    pr = np.exp(x - x.max())
    pr /= pr.sum()
    return int(np.argmax(pr / expo))


# ---------------------------------------------------------------------------------------------
# the HIP sampler's specification, bit for bit
# ---------------------------------------------------------------------------------------------
def philox4x32(counter, key, rounds: int = 10) -> np.ndarray:
    """Philox4x32 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11).
    ``counter`` [..., 4] and ``key`` [..., 2] uint32; returns [..., 4] uint32."""
    c = np.array(counter, dtype=np.uint64) & np.uint64(0xFFFFFFFF)
    k = np.array(key, dtype=np.uint64) & np.uint64(0xFFFFFFFF)
    c0, c1, c2, c3 = (c[..., i].copy() for i in range(4))
    k0, k1 = k[..., 0].copy(), k[..., 1].copy()
    M0, M1, MASK = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57), np.uint64(0xFFFFFFFF)
    for _ in range(rounds):
        p0, p1 = M0 * c0, M1 * c2
        c0, c1, c2, c3 = ((p1 >> np.uint64(32)) ^ c1 ^ k0) & MASK, p1 & MASK, ((p0 >> np.uint64(32)) ^ c3 ^ k1) & MASK, p0 & MASK
        k0 = (k0 + np.uint64(0x9E3779B9)) & MASK
        k1 = (k1 + np.uint64(0xBB67AE85)) & MASK
    return np.stack([c0, c1, c2, c3], axis=-1).astype(np.uint32)


def exp32(d: np.ndarray) -> np.ndarray:
    """exp(d), |d| <= 32, in float32 operations only (no fused multiply-add)."""
    d = d.astype(F)
    n = np.rint(d * F(1.44269502162933349609375))
    r = (d - n * F(0.693145751953125)) - n * F(1.428606765330187045037746429443359375e-06)
    p = np.full_like(r, F(1.0) / F(5040.0))
    for c in (F(1.0) / F(720.0), F(1.0) / F(120.0), F(1.0) / F(24.0), F(1.0) / F(6.0), F(0.5), F(1.0), F(1.0)):
        p = p * r + c
    bits = p.view(np.int32) + n.astype(np.int32) * np.int32(1 << 23)
    return bits.view(F)


def neg_log_uniform(n: np.ndarray) -> np.ndarray:
    """-log((2 n + 1) / 2^33) for uint32 ``n`` in float32 operations only."""
    f = (np.uint64(2) * n.astype(np.uint64) + np.uint64(1)).astype(F)  # rounds to nearest even
    b = f.view(np.uint32)
    e = (b >> np.uint32(23)).astype(np.int32) - 127
    m = ((b & np.uint32(0x007FFFFF)) | np.uint32(0x3F800000)).view(F)
    big = m > F(1.41421353816986083984375)
    m = np.where(big, m * F(0.5), m)
    e = e + big.astype(np.int32)
    s = (m - F(1.0)) / (m + F(1.0))
    s2 = s * s
    q = np.full_like(s, F(1.0) / F(9.0))
    for c in (F(1.0) / F(7.0), F(1.0) / F(5.0), F(1.0) / F(3.0), F(1.0)):
        q = q * s2 + c
    logm = (F(2.0) * s) * q
    return (33 - e).astype(F) * F(0.693147182464599609375) - logm


def float_key(x: np.ndarray) -> np.ndarray:
    b = x.astype(F).view(np.uint32)
    return np.where(b & np.uint32(0x80000000), ~b, b | np.uint32(0x80000000)).astype(np.uint32)


def scaled_logits(logits: np.ndarray, temperature: float) -> np.ndarray:
    x = logits.astype(F)
    if F(temperature) != F(1.0):
        x = x * (F(1.0) / F(temperature))
    return x


def kept_mask_spec(x: np.ndarray, top_k, top_p) -> np.ndarray:
    """The kernel's masks for one row of scaled logits ``x`` (float32): top-k by key, then top-p by
    integer mass; also drops tokens more than 32 below the maximum."""
    V = x.size
    key = float_key(x)
    thr = np.uint32(0)
    if top_k is not None and 0 < top_k < V:
        thr = np.sort(key)[V - top_k]
    d = x - x.max()
    live = d >= CUTOFF
    if top_p is not None and F(top_p) < F(1.0):
        ok = live & (key >= thr)
        w = np.zeros(V, dtype=np.uint64)
        w[ok] = (exp32(d[ok]) * F(4294967296.0)).astype(np.uint64)
        Q = int(w.sum())
        L = int(np.float64(F(1.0) - F(top_p)) * np.float64(Q))
        order = np.argsort(key, kind="stable")
        ks, ws = key[order], np.cumsum(w[order])  # < 2^50: exact in uint64
        # inclusive mass of a key class = cumulative mass at the last element of the class
        last = np.r_[ks[1:] != ks[:-1], True]
        cls_keys, cls_mass = ks[last], ws[last]
        i = int(np.searchsorted(cls_mass, np.uint64(L), side="right"))  # first class with mass > L
        thr = max(thr, cls_keys[min(i, cls_keys.size - 1)])
    return live & (key >= thr)


def sample_tokens_ref(logits: np.ndarray, temperature: float, top_k, top_p, seeds, positions) -> np.ndarray:
    """Tokens the HIP sampler must return for ``logits`` [B, V] (any float dtype numpy can widen)."""
    B, V = logits.shape
    out = np.zeros(B, dtype=np.int64)
    groups = (V + 3) // 4
    for b in range(B):
        x = scaled_logits(logits[b], temperature)
        keep = kept_mask_spec(x, top_k, top_p)
        seed, pos = int(seeds[b]) & (2**64 - 1), int(positions[b]) & (2**64 - 1)
        ctr = np.zeros((groups, 4), dtype=np.uint64)
        ctr[:, 0] = np.arange(groups)
        ctr[:, 1], ctr[:, 2] = pos & 0xFFFFFFFF, pos >> 32
        rnd = philox4x32(ctr, np.array([seed & 0xFFFFFFFF, seed >> 32], dtype=np.uint64)).reshape(-1)[:V]
        score = np.full(V, np.inf, dtype=F)
        score[keep] = neg_log_uniform(rnd[keep]) * exp32((x.max() - x)[keep])
        out[b] = int(np.argmin(score))  # first index on ties
    return out
