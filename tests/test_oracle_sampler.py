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


def test_oracle_arithmetic_is_the_kernel_source_arithmetic(tmp_path):
    """The sampler's scalar arithmetic (order-preserving keys, exp, -log of a uniform, Philox) is plain C++ inside
    vexact_amd/csrc/sampler.hip. Its text is compiled here for the host, unchanged, and compared bit for bit with the numpy
    restatement: what the GPU tests compare token ids against is then the shipped source's arithmetic, not a look-alike."""
    import ctypes
    import os
    import subprocess

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "vexact_amd", "csrc", "sampler.hip")).read()
    start = text.index("__device__ __forceinline__ uint32_t float_key(float x)")
    end = text.index("struct SampleParams {")
    body = text[start:end]
    for name in ("float_key", "exp32", "neg_log_uniform", "philox4x32"):
        assert f" {name}(" in body
    src = tmp_path / "sampler_math.cpp"
    src.write_text(
        "#include <math.h>\n#include <stdint.h>\n#define __device__\n#define __forceinline__ inline\n"
        "struct uint4 { uint32_t x, y, z, w; };\n"
        "static inline uint4 make_uint4(uint32_t x, uint32_t y, uint32_t z, uint32_t w) { return uint4{x, y, z, w}; }\n"
        + body +
        'extern "C" {\n'
        "void k_float_key(const float* x, uint32_t* o, int64_t n) { for (int64_t i = 0; i < n; i++) o[i] = float_key(x[i]); }\n"
        "void k_exp32(const float* x, float* o, int64_t n) { for (int64_t i = 0; i < n; i++) o[i] = exp32(x[i]); }\n"
        "void k_neg_log_uniform(const uint32_t* x, float* o, int64_t n) { for (int64_t i = 0; i < n; i++) o[i] = neg_log_uniform(x[i]); }\n"
        "void k_philox(const uint32_t* c, const uint32_t* k, uint32_t* o, int64_t n) {\n"
        "  for (int64_t i = 0; i < n; i++) { const uint4 r = philox4x32(uint4{c[4 * i], c[4 * i + 1], c[4 * i + 2], c[4 * i + 3]}, k[2 * i], k[2 * i + 1]);\n"
        "    o[4 * i] = r.x; o[4 * i + 1] = r.y; o[4 * i + 2] = r.z; o[4 * i + 3] = r.w; } }\n"
        "}\n")
    so = tmp_path / "sampler_math.so"
    subprocess.run(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-ffp-contract=off", "-o", str(so), str(src)], check=True)
    lib = ctypes.CDLL(str(so))
    rng = np.random.default_rng(5)
    P = lambda a: a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    n = 400_000
    # keys: any float, including the signed zeros, infinities and subnormals
    x = np.concatenate([rng.standard_normal(n).astype(np.float32) * 50, rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32).view(np.float32),
                        np.array([0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-45], dtype=np.float32)])
    x = x[~np.isnan(x)]
    out = np.empty(x.size, dtype=np.uint32)
    lib.k_float_key(P(x), P(out), ctypes.c_int64(x.size))
    assert np.array_equal(out, S.float_key(x))
    # exp on [-32, 0] (what the kernel feeds it) and a little beyond
    d = np.concatenate([-rng.random(n).astype(np.float32) * 32, np.linspace(-33, 1, 4097, dtype=np.float32), np.array([0.0, -32.0], dtype=np.float32)])
    out = np.empty(d.size, dtype=np.float32)
    lib.k_exp32(P(d), P(out), ctypes.c_int64(d.size))
    assert np.array_equal(out.view(np.uint32), S.exp32(d).view(np.uint32))
    # -log u for every kind of 32-bit draw
    u = np.concatenate([rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32), np.array([0, 1, 2, 2**31 - 1, 2**31, 2**32 - 1], dtype=np.uint32),
                        (np.uint32(1) << np.arange(32, dtype=np.uint32))])
    out = np.empty(u.size, dtype=np.float32)
    lib.k_neg_log_uniform(P(u), P(out), ctypes.c_int64(u.size))
    assert np.array_equal(out.view(np.uint32), S.neg_log_uniform(u).view(np.uint32))
    # Philox on random counters and keys
    c = rng.integers(0, 2**32, (20_000, 4), dtype=np.uint64).astype(np.uint32)
    k = rng.integers(0, 2**32, (20_000, 2), dtype=np.uint64).astype(np.uint32)
    out = np.empty_like(c)
    lib.k_philox(P(np.ascontiguousarray(c)), P(np.ascontiguousarray(k)), P(out), ctypes.c_int64(c.shape[0]))
    assert np.array_equal(out, S.philox4x32(c, k))
