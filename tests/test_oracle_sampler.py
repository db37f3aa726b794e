"""Pins the sampler restatement: Philox against its published known-answer vectors, the two
polynomials against numpy's exp / log, the integer-mass top-k / top-p rule against the reference's
sort-and-cumsum formula, the fused race against ``argmax(probs / q)`` and against the softmax
distribution."""

import numpy as np
import pytest

from oracle import sampler as S


def test_philox_known_answers():
    # Random123 kat_vectors, philox4x32 with 10 rounds: counter, key -> output
    kat = [
        ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
        ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
        ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
         (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
    ]
    for ctr, key, want in kat:
        got = S.philox4x32(np.array(ctr, dtype=np.uint64), np.array(key, dtype=np.uint64))
        assert tuple(int(v) for v in got) == want
    # vectorised over counters == one at a time
    ctrs = np.arange(40, dtype=np.uint64).reshape(10, 4)
    many = S.philox4x32(ctrs, np.array([7, 9], dtype=np.uint64))
    for i in range(10):
        assert np.array_equal(many[i], S.philox4x32(ctrs[i], np.array([7, 9], dtype=np.uint64)))


def test_polynomials_track_libm():
    d = np.linspace(-32, 32, 200001).astype(np.float32)
    rel = np.abs(S.exp32(d).astype(np.float64) / np.exp(d.astype(np.float64)) - 1)
    assert rel.max() < 4e-7
    assert S.exp32(np.float32([0.0]))[0] == 1.0
    rng = np.random.default_rng(0)
    n = np.concatenate([rng.integers(0, 2**32, 200000, dtype=np.uint64).astype(np.uint32),
                        np.array([0, 1, 2, 2**31 - 1, 2**31, 2**32 - 2, 2**32 - 1], dtype=np.uint32)])
    want = -np.log((2.0 * n.astype(np.float64) + 1.0) / 2.0**33)
    got = S.neg_log_uniform(n).astype(np.float64)
    assert (got >= 0).all()
    big = want > 0.25
    assert (np.abs(got[big] / want[big] - 1)).max() < 2e-6      # relative accuracy away from u = 1
    assert np.abs(got[~big] - want[~big]).max() < 1e-7            # float32(2n+1) has 24 bits: absolute near u = 1


@pytest.mark.parametrize("k,p", [(None, 0.9), (50, 1.0), (50, 0.9), (5, 0.5), (None, 0.99), (200, 0.3), (1, 0.9)])
def test_mass_rule_equals_sort_and_cumsum_rule(k, p):
    rng = np.random.default_rng(3)
    for trial in range(6):
        V = int(rng.integers(300, 3000))
        x = (rng.standard_normal(V) * 3).astype(np.float32)
        assert np.unique(x).size == V                             # tie-free
        want = S.apply_top_k_top_p_ref(x, k, p)
        got = S.kept_mask_spec(x, k, p)
        if not np.array_equal(got, want):
            # only a token whose cumulative probability sits on the limit (to rounding) may differ
            diff = np.flatnonzero(got != want)
            assert diff.size == 1
            order = np.argsort(x.astype(np.float64), kind="stable")
            xs = np.where(want | got, x, -np.inf)[order].astype(np.float64)
            e = np.exp(xs - xs.max())
            cum = np.cumsum(e / e.sum())[np.flatnonzero(order == diff[0])[0]]
            assert abs(cum - (1 - p)) < 1e-6
        assert got.sum() >= 1


def test_ties_are_kept_or_masked_together_and_cutoff_applies():
    x = np.float32([0.0, 0.0, 0.0, 0.0, -1.0, -1.0, -50.0])
    keep = S.kept_mask_spec(x, None, 0.5)        # the -1 class holds 2e^-1/(4+2e^-1) = 15.5 % <= 50 %: masked
    assert keep.tolist() == [True] * 4 + [False] * 3
    keep = S.kept_mask_spec(x, None, 0.9)        # 15.5 % > 10 %: kept, both of them
    assert keep.tolist() == [True] * 6 + [False]
    assert S.kept_mask_spec(x, None, 1.0).tolist() == [True] * 6 + [False]   # 50 below the maximum: never sampled
    assert S.kept_mask_spec(x, 2, 1.0).tolist() == [True] * 4 + [False] * 3  # ties at the k-th value all stay
    assert S.kept_mask_spec(x, 5, 1.0).tolist() == [True] * 6 + [False]


def test_race_equals_argmax_of_probs_over_exponentials():
    rng = np.random.default_rng(4)
    agree = 0
    for trial in range(200):
        V = 257
        x = (rng.standard_normal((1, V)) * 2).astype(np.float32)
        seed, pos = int(rng.integers(0, 2**62)), int(rng.integers(0, 2**40))
        tok = int(S.sample_tokens_ref(x, 1.0, 20, 0.8, [seed], [pos])[0])
        keep = S.kept_mask_spec(x[0], 20, 0.8)
        ctr = np.zeros(((V + 3) // 4, 4), dtype=np.uint64)
        ctr[:, 0] = np.arange((V + 3) // 4)
        ctr[:, 1], ctr[:, 2] = pos & 0xFFFFFFFF, pos >> 32
        rnd = S.philox4x32(ctr, np.array([seed & 0xFFFFFFFF, seed >> 32], dtype=np.uint64)).reshape(-1)[:V]
        expo = -np.log((2.0 * rnd.astype(np.float64) + 1.0) / 2.0**33)
        agree += tok == S.race_ref(x[0], keep, expo)
        assert keep[tok]
    assert agree >= 199          # float32 vs float64 scores can swap a photo finish


def test_sampled_frequencies_follow_softmax():
    x = np.float32([[1.0, 0.0, -1.0, 2.0, 0.5, -3.0, 1.5, 0.25]])
    n = 20000
    logits = np.repeat(x, n, axis=0)
    for temperature in (1.0, 0.7):
        toks = S.sample_tokens_ref(logits, temperature, None, 1.0, np.full(n, 12345), np.arange(n))
        pr = np.exp(x[0].astype(np.float64) / temperature)
        pr /= pr.sum()
        freq = np.bincount(toks, minlength=8) / n
        assert (np.abs(freq - pr) < 4.5 * np.sqrt(pr * (1 - pr) / n)).all(), (freq, pr)
    # top-k = 3 renormalises over the three largest
    toks = S.sample_tokens_ref(logits, 1.0, 3, 1.0, np.full(n, 777), np.arange(n))
    pr = np.exp(x[0].astype(np.float64)) * np.isin(np.arange(8), [3, 6, 0])
    pr /= pr.sum()
    freq = np.bincount(toks, minlength=8) / n
    assert (np.abs(freq - pr) < 4.5 * np.sqrt(pr * (1 - pr) / n + 1e-12)).all()


def test_token_depends_on_seed_and_position_only():
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((6, 500)) * 2).astype(np.float32)
    seeds, pos = rng.integers(0, 2**62, 6), rng.integers(0, 10**6, 6)
    a = S.sample_tokens_ref(x, 0.9, 40, 0.95, seeds, pos)
    perm = np.array([3, 0, 5, 1, 4, 2])
    b = S.sample_tokens_ref(x[perm], 0.9, 40, 0.95, seeds[perm], pos[perm])
    assert np.array_equal(b, a[perm])
    c = S.sample_tokens_ref(x, 0.9, 40, 0.95, seeds, pos + 1)
    assert not np.array_equal(a, c)
