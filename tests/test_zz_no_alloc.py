"""The entry point that allocates nothing: ``vx_logprobs_static`` keeps its chunk partials in an array
inside the library's device image instead of a caller's workspace. Called through the C ABI and compared
bit for bit with ``vx_logprobs`` on two calls in a row, the second smaller than the first (the array keeps
the first call's contents), and beyond its size limit."""

import pytest
import torch

from tests.util import assert_bitwise

pytestmark = pytest.mark.gpu


def _both(lib, logits, labels):
    rows, n = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    dt = {torch.float32: 0, torch.bfloat16: 1}[logits.dtype]
    lab = labels.data_ptr() if labels is not None else None
    ws = torch.empty(max(16, lib.vx_log_softmax_workspace_bytes(rows, n)), dtype=torch.uint8, device="cuda")
    out_a = torch.full((rows,), 3.0, dtype=torch.float32, device="cuda")
    tok_a = torch.full((rows,), -7, dtype=torch.int64, device="cuda")
    out_b, tok_b = out_a.clone(), tok_a.clone()
    torch.cuda.synchronize()
    rc = lib.vx_logprobs(logits.data_ptr(), lab, out_a.data_ptr(), tok_a.data_ptr(), dt, rows, n, logits.stride(0),
                         ws.data_ptr(), ws.numel(), stream)
    assert rc == 0
    rc = lib.vx_logprobs_static(logits.data_ptr(), lab, out_b.data_ptr(), tok_b.data_ptr(), dt, rows, n,
                                logits.stride(0), stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return (out_a.cpu(), tok_a.cpu()), (out_b.cpu(), tok_b.cpu())


def test_logprobs_static_matches_logprobs_on_two_calls_in_a_row():
    from vexact_amd import _lib

    lib = _lib.load()
    g = torch.Generator().manual_seed(12)
    # first call: the headline shape (256 rows of a 151936-entry vocabulary, bf16), greedy tokens
    big = (torch.randn(256, 151936, generator=g) * 3).to(torch.bfloat16).cuda()
    (lp_a, tok_a), (lp_b, tok_b) = _both(lib, big, None)
    assert_bitwise(lp_b, lp_a, "first call: logprobs")
    assert torch.equal(tok_b, tok_a)
    assert bool(torch.isfinite(lp_b).all()) and bool((tok_b >= 0).all())
    # second call, smaller, fp32, given labels, odd row length: the array still holds the first call's partials
    small = torch.randn(7, 5000, generator=g).cuda()
    labels = torch.randint(0, 5000, (7,), generator=g).cuda()
    (lp_a, tok_a), (lp_b, tok_b) = _both(lib, small, labels)
    assert_bitwise(lp_b, lp_a, "second call: logprobs")
    assert torch.equal(tok_b, labels.cpu())
    want = torch.log_softmax(small.cpu(), -1).gather(1, labels.cpu()[:, None])[:, 0]
    assert float((lp_b - want).abs().max()) <= 1e-5
    # third: one row
    (lp_a, _), (lp_b, _) = _both(lib, big[3:4], None)
    assert_bitwise(lp_b, lp_a, "one row")


def test_logprobs_static_rejects_what_does_not_fit():
    from vexact_amd import _lib

    lib = _lib.load()
    x = torch.zeros(8, 16, device="cuda")
    out = torch.zeros(8, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    # 65536 rows x 2 chunks x 16 bytes = 2 MiB of partials > 1 MiB: refused before any launch
    assert lib.vx_logprobs_static(x.data_ptr(), None, out.data_ptr(), None, 0, 65536, 8192, 8192, s) == -3
    assert b"workspace" in lib.vx_status_string(-3)
    assert lib.vx_logprobs_static(x.data_ptr(), None, None, None, 0, 8, 16, 16, s) == -1  # no output pointer
    assert lib.vx_logprobs_static(x.data_ptr(), None, out.data_ptr(), None, 0, 0, 16, 16, s) == 0  # nothing to do
    torch.cuda.synchronize()
