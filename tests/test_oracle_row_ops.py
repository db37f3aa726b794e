"""Pins the row-op / GEMM oracle against fp64 brute force, closed forms and library routines."""

import math

import torch

from oracle import row_ops as O


def _gen(shape, seed, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def test_matmul_ref_brute_force_and_exact_integers():
    a, b, bias = _gen((5, 24), 1, torch.bfloat16), _gen((24, 7), 2, torch.bfloat16), _gen((7,), 3, torch.bfloat16)
    got = O.matmul_ref(a, b, bias)
    for i in range(5):
        for j in range(7):
            acc = sum(float(a[i, k]) * float(b[k, j]) for k in range(24)) + float(bias[j])
            want = torch.tensor(acc, dtype=torch.float64).to(torch.bfloat16)
            near = abs(float(got[i, j]) - acc) <= 2 ** -8 * abs(acc) + 1e-6
            assert got[i, j] == want or near
    # small integers: every product and sum is exact, so the result is exact
    ai = torch.randint(-4, 5, (6, 16), generator=torch.Generator().manual_seed(4)).to(torch.bfloat16)
    bi = torch.randint(-4, 5, (16, 3), generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    assert torch.equal(O.matmul_ref(ai, bi).float(), (ai.double() @ bi.double()).float())
    # a transposed operand must not change anything (index mistakes show up here)
    assert torch.equal(O.matmul_ref(a, b), O.matmul_ref(a, b.t().contiguous().t()))


def test_mean_dim_ref():
    x = _gen((3, 10, 4), 6)
    for dim in (0, 1, 2, -1):
        want = x.double().mean(dim).float()
        torch.testing.assert_close(O.mean_dim_ref(x, dim), want, atol=1e-6, rtol=1e-6)
    assert O.mean_dim_ref(x, 1, keepdim=True).shape == (3, 1, 4)
    c = torch.full((4, 9), 2.5)
    assert torch.equal(O.mean_dim_ref(c, 1), torch.full((4,), 2.5))
    xi = torch.arange(12, dtype=torch.int64).reshape(3, 4)
    assert O.mean_dim_ref(xi, 1).dtype == torch.float32 and torch.equal(O.mean_dim_ref(xi, 1), torch.tensor([1.5, 5.5, 9.5]))


def test_rms_norm_refs():
    x, w = _gen((4, 64), 7, torch.bfloat16), (1 + 0.1 * _gen((64,), 8)).to(torch.bfloat16)
    one, two = O.rms_norm_ref(x, w, 1e-6), O.hf_rms_norm_ref(x, w, 1e-6)
    xd, wd = x.double(), w.double()
    want = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-6) * wd
    assert (one.double() - want).abs().max() <= 2 ** -8 * want.abs().max()
    assert (two.double() - want).abs().max() <= 2 ** -7 * want.abs().max()
    # the two rounding variants differ by at most one bf16 ulp
    i1 = one.view(torch.int16).int()
    i2 = two.view(torch.int16).int()
    assert (i1 - i2).abs().max() <= 1
    # constant row, unit weight: x / sqrt(x^2 + eps) = sign(x) up to eps
    c = torch.full((2, 32), -3.0, dtype=torch.bfloat16)
    assert torch.equal(O.rms_norm_ref(c, torch.ones(32, dtype=torch.bfloat16)), torch.full((2, 32), -1.0, dtype=torch.bfloat16))
    assert torch.equal(O.hf_rms_norm_ref(c, torch.ones(32, dtype=torch.bfloat16)), torch.full((2, 32), -1.0, dtype=torch.bfloat16))
    # scaling the weight scales the output (weight enters linearly, powers of two are exact)
    assert torch.equal(O.rms_norm_ref(x, w * 2).float(), O.rms_norm_ref(x, w).float() * 2)


def test_log_softmax_and_logprobs_refs():
    x = _gen((6, 1000), 9, scale=4.0)
    got = O.log_softmax_ref(x)
    torch.testing.assert_close(got, torch.log_softmax(x, -1), atol=1e-5, rtol=0)
    torch.testing.assert_close(got.double().exp().sum(-1), torch.ones(6, dtype=torch.float64), atol=1e-5, rtol=0)
    torch.testing.assert_close(O.log_softmax_ref(x + 3.0), got, atol=2e-5, rtol=0)  # shift invariance
    labels = torch.tensor([0, 999, 5, 17, 400, 3])
    lp = O.logprobs_ref(x, labels)
    for i in range(6):
        want = float(x[i, labels[i]]) - math.log(sum(math.exp(float(v)) for v in x[i]))
        assert abs(float(lp[i]) - want) < 1e-4
    # the fallback formula the reference states: gather of log_softmax
    assert torch.equal(lp, torch.log_softmax(x, -1).gather(-1, labels[:, None]).squeeze(-1)) or (
        (lp - torch.log_softmax(x, -1).gather(-1, labels[:, None]).squeeze(-1)).abs().max() < 1e-5)
