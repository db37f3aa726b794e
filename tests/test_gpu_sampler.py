"""GPU parity of the sampler: the kernel against its CPU restatement bit for bit (integer work),
the reference's own sampling properties (tests/test_inferencer_sampling.py:88-200: error cases,
repeatability, request-order invariance), batch invariance and the sampled distribution."""

import types

import numpy as np
import pytest
import torch

from oracle import sampler as OS

pytestmark = pytest.mark.gpu

from vexact_amd import ops  # noqa: E402
from vexact_amd.sampler import Sampler  # noqa: E402


def _cfg(seed=None, **kw):
    c = types.SimpleNamespace(do_sample=True, temperature=1.0, top_k=None, top_p=1.0)
    c.__dict__.update(kw)
    if seed is not None:
        c.seed = seed
    return c


def _run(logits, temperature, k, p, seeds, pos):
    dev = logits.device
    return ops.sample_tokens(logits, temperature, k, p, torch.as_tensor(np.asarray(seeds), dtype=torch.int64).to(dev),
                             torch.as_tensor(np.asarray(pos), dtype=torch.int64).to(dev)).cpu().numpy()


@pytest.mark.parametrize("B,V,dtype,temperature,k,p", [
    (4, 5, torch.float32, 1.0, None, 1.0),
    (4, 5, torch.float32, 1.0, 2, 0.7),
    (6, 1000, torch.float32, 0.7, 50, 0.9),
    (6, 1000, torch.bfloat16, 1.0, None, 0.9),
    (5, 4099, torch.bfloat16, 1.3, 64, 1.0),        # odd row pitch: unaligned rows, ragged tail
    (5, 4099, torch.float32, 1.0, 4099, 0.5),       # k >= V is off
    (3, 151936, torch.bfloat16, 1.0, None, 1.0),    # plain sampling at the full vocabulary
    (3, 151936, torch.bfloat16, 0.8, 50, 0.9),
    (2, 151936, torch.float32, 1.0, None, 0.95),
])
def test_kernel_equals_cpu_restatement(B, V, dtype, temperature, k, p):
    g = torch.Generator().manual_seed(V * 7 + B)
    x = (torch.randn(B, V, generator=g) * 2.5).to(dtype)
    rng = np.random.default_rng(V)
    seeds, pos = rng.integers(0, 2**62, B), rng.integers(0, 2**33, B)
    print(f"[case] sample B={B} V={V} {dtype} T={temperature} k={k} p={p}", flush=True)
    got = _run(x.cuda(), temperature, k, p, seeds, pos)
    want = OS.sample_tokens_ref(x.float().numpy(), temperature, k, p, seeds, pos)
    assert np.array_equal(got, want)


def test_ties_and_peaked_rows():
    # many equal logits (bf16 logits tie constantly), a one-hot-like row, and a row with a lone survivor
    V = 2048
    x = torch.zeros(4, V)
    x[0, ::3] = 1.0
    x[1, 77] = 40.0                       # everything else is more than 32 below: token 77 for sure
    x[2] = torch.arange(V) % 7
    x[3, 5] = 3.0
    seeds, pos = [1, 2, 3, 4], [10, 11, 12, 13]
    for k, p in ((None, 0.5), (10, 1.0), (10, 0.2), (1, 1.0)):
        got = _run(x.cuda(), 1.0, k, p, seeds, pos)
        want = OS.sample_tokens_ref(x.numpy(), 1.0, k, p, seeds, pos)
        assert np.array_equal(got, want), (k, p)
        assert got[1] == 77
        if k == 1:
            assert got[3] == 5


def test_row_alone_equals_row_in_batch_and_any_order():
    V, B = 32000, 256
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(B, V, generator=g) * 3).to(torch.bfloat16).cuda()
    rng = np.random.default_rng(2)
    seeds, pos = rng.integers(0, 2**62, B), rng.integers(0, 5000, B)
    full = _run(x, 0.9, 50, 0.9, seeds, pos)
    for r in (0, 17, 255):
        assert _run(x[r : r + 1], 0.9, 50, 0.9, seeds[r : r + 1], pos[r : r + 1])[0] == full[r]
    perm = rng.permutation(B)
    assert np.array_equal(_run(x[torch.from_numpy(perm).cuda()], 0.9, 50, 0.9, seeds[perm], pos[perm]), full[perm])
    assert np.array_equal(_run(x, 0.9, 50, 0.9, seeds, pos), full)                 # repeatable
    assert not np.array_equal(_run(x, 0.9, 50, 0.9, seeds, pos + 1), full)         # the position matters
    assert not np.array_equal(_run(x, 0.9, 50, 0.9, seeds + 1, pos), full)         # and the seed


def test_sampled_frequencies_follow_softmax_on_the_gpu():
    x = torch.tensor([[1.0, 0.0, -1.0, 2.0, 0.5, -3.0, 1.5, 0.25]])
    n = 40000
    toks = _run(x.repeat(n, 1).cuda(), 1.0, None, 1.0, np.full(n, 99), np.arange(n))
    pr = torch.softmax(x[0].double(), 0).numpy()
    freq = np.bincount(toks, minlength=8) / n
    assert (np.abs(freq - pr) < 4.5 * np.sqrt(pr * (1 - pr) / n)).all(), (freq, pr)


def test_sampler_interface_properties():
    s = Sampler()
    dev = "cuda"
    # error cases of the reference (checked before any device work)
    logits = torch.randn(2, 16)
    cfgs = [_cfg(top_k=4), _cfg(top_k=4)]
    cfgs[0].seed = 1234
    with pytest.raises(ValueError, match="every request in the batch"):
        s.batch_sample_token(logits, cfgs, torch.arange(2))
    for c in cfgs:
        c.seed = 1234
    with pytest.raises(ValueError, match="sampling_positions must be set"):
        s.batch_sample_token(logits, cfgs)
    # seeded: repeatable with other random work in between, and request-order invariant
    B, V = 8, 4096
    logits = torch.empty(B, V, device=dev).uniform_(-1.0, 1.0)
    positions = torch.arange(17, 17 + B, device=dev)
    for top_k, top_p in ((50, 1.0), (50, 0.9)):
        cfgs = [_cfg(seed=1234 + i, top_k=top_k, top_p=top_p) for i in range(B)]
        first = s.batch_sample_token(logits.clone(), cfgs, positions)
        torch.empty(1024, device=dev).exponential_()
        assert torch.equal(s.batch_sample_token(logits.clone(), cfgs, positions), first)
        perm = torch.tensor([3, 0, 7, 1, 4, 2, 6, 5], device=dev)
        permuted = s.batch_sample_token(logits.index_select(0, perm).clone(), [cfgs[i] for i in perm.tolist()],
                                        positions.index_select(0, perm))
        assert torch.equal(permuted, first.index_select(0, perm))
        assert first.dtype == torch.long and bool(((first >= 0) & (first < V)).all())
        # every sampled token is inside the top-k set
        topk = logits.topk(top_k, dim=-1).indices
        assert bool((topk == first[:, None]).any(dim=1).all())
    # unseeded: follows torch's default generator, greedy ignores it
    cfgs = [_cfg(top_k=0, top_p=0.9) for _ in range(B)]
    torch.manual_seed(42)
    a = s.batch_sample_token(logits, cfgs)
    torch.manual_seed(42)
    assert torch.equal(s.batch_sample_token(logits, cfgs), a)
    for greedy in (_cfg(do_sample=False), _cfg(temperature=0.0), _cfg(top_p=0)):
        assert torch.equal(s.batch_sample_token(logits, [greedy] * B), logits.argmax(-1))
