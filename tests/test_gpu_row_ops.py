"""GPU parity: mean / RMSNorm / log_softmax / logprobs against the CPU oracle, and row invariance.

Restates the reference formulas of vexact/batch_invariant_ops/batch_invariant_ops.py:231-381,637-669
and the permutation test tests/batch_invariant_ops/test_batch_invariance.py:131-157.
"""

import pytest
import torch

from oracle import row_ops as O
from tests.util import assert_bf16_close, assert_bitwise

pytestmark = pytest.mark.gpu

from vexact_amd import ops  # noqa: E402
from vexact_amd.batch_invariant_ops import batch_invariant_rms_norm, log_softmax, mean_dim  # noqa: E402
from vexact_amd.batch_invariant_ops.standalone_logprobs import logprobs_from_logits_flash_attn  # noqa: E402


def _gen(shape, seed, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("shape,dim", [((7, 2048), -1), ((3, 5, 128), -1), ((4, 33, 6), 1), ((2, 1000, 3), 1), ((5, 700), 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mean_dim_matches_oracle(shape, dim, dtype):
    x = _gen(shape, 1, dtype)
    for keepdim in (False, True):
        got = mean_dim(x.cuda(), dim, keepdim=keepdim).cpu()
        ref = O.mean_dim_ref(x, dim, keepdim=keepdim)
        assert got.shape == ref.shape and got.dtype == ref.dtype
        # fp32 sums in a different order: a few fp32 ulps of the sum of |x|
        torch.testing.assert_close(got.float(), ref.float(), atol=2e-6 if dtype == torch.float32 else 1e-2, rtol=1e-5 if dtype == torch.float32 else 1e-2)


def test_mean_dim_int_input_and_row_invariance():
    xi = torch.arange(24, dtype=torch.int32).reshape(4, 6)
    got = mean_dim(xi.cuda(), 1).cpu()
    assert got.dtype == torch.float32
    torch.testing.assert_close(got, xi.float().mean(1), atol=0, rtol=0)
    x = _gen((64, 2048), 2).pow(2)
    full = mean_dim(x.cuda(), -1, keepdim=True)
    for m in (1, 7):
        assert_bitwise(mean_dim(x[:m].cuda(), -1, keepdim=True), full[:m], f"mean rows {m}")
    assert_bitwise(mean_dim(x[13:14].cuda(), -1, keepdim=True), full[13:14], "mean single row 13")


@pytest.mark.parametrize("n", [128, 2048, 4096, 1000])
def test_rms_norm_both_roundings(n):
    x = _gen((9, n), 3, torch.bfloat16)
    w = (1.0 + 0.02 * _gen((n,), 4)).to(torch.bfloat16)
    one = batch_invariant_rms_norm(x.cuda(), w.cuda(), 1e-6).cpu()
    assert_bf16_close(one, O.rms_norm_ref(x, w, 1e-6), max_ulp=1, what="one-rounding rms_norm")
    two = ops.rms_norm(x.cuda(), w.cuda(), 1e-6, hf_two_rounding=True).cpu()
    assert_bf16_close(two, O.hf_rms_norm_ref(x, w, 1e-6), max_ulp=1, what="two-rounding rms_norm")
    # fp32 in/out
    xf = x.float()
    got = ops.rms_norm(xf.cuda(), w.float().cuda(), 1e-6).cpu()
    torch.testing.assert_close(got, O.rms_norm_ref(xf, w.float(), 1e-6), atol=1e-5, rtol=1e-5)


def test_rms_norm_row_invariance_and_residual():
    x = _gen((64, 2048), 5, torch.bfloat16)
    r = _gen((64, 2048), 6, torch.bfloat16)
    w = (1.0 + 0.02 * _gen((2048,), 7)).to(torch.bfloat16)
    xg, rg, wg = x.cuda(), r.cuda(), w.cuda()
    for mode in (False, True):
        full = ops.rms_norm(xg, wg, 1e-6, hf_two_rounding=mode)
        for m in (1, 7):
            assert_bitwise(ops.rms_norm(xg[:m], wg, 1e-6, hf_two_rounding=mode), full[:m], f"rms rows {m}")
        assert_bitwise(ops.rms_norm(xg[40:41], wg, 1e-6, hf_two_rounding=mode), full[40:41], "rms row 40")
    # fused residual == separate bf16 add, and the sum is written (also in place over x)
    s = torch.empty_like(xg)
    y = ops.rms_norm(xg, wg, 1e-6, hf_two_rounding=True, residual=rg, sum_out=s)
    ssum = (x.float() + r.float()).to(torch.bfloat16)
    assert_bitwise(s, ssum, "residual sum")
    assert_bitwise(y, ops.rms_norm(ssum.cuda(), wg, 1e-6, hf_two_rounding=True), "fused residual norm")
    x2 = xg.clone()
    y2 = ops.rms_norm(x2, wg, 1e-6, hf_two_rounding=True, residual=rg, sum_out=x2)
    assert_bitwise(x2, ssum, "in-place residual sum")
    assert_bitwise(y2, y, "in-place fused residual norm")


def test_rms_norm_head_rows_match_unfused_mean_path():
    # HF RMSNorm under the overrides: x.float().pow(2).mean(-1) through mean_dim, then torch glue
    x = _gen((6, 16, 128), 8, torch.bfloat16).cuda()
    w = (1.0 + 0.02 * _gen((128,), 9)).to(torch.bfloat16).cuda()
    xf = x.float()
    var = mean_dim(xf.pow(2), -1, keepdim=True)
    glue = w * (xf * torch.rsqrt(var + 1e-6)).to(torch.bfloat16)
    fused = ops.rms_norm(x, w, 1e-6, hf_two_rounding=True)
    assert_bf16_close(fused, glue, max_ulp=1, what="fused vs mean_dim + torch glue")


@pytest.mark.parametrize("rows,n", [(7, 151936), (3, 4096), (5, 1000), (2, 8193)])
def test_log_softmax_matches_oracle_and_is_row_invariant(rows, n):
    x = _gen((rows, n), 10, scale=3.0)
    got = log_softmax(x.cuda(), dim=-1)
    ref = O.log_softmax_ref(x)
    torch.testing.assert_close(got.cpu(), ref, atol=2e-5, rtol=0)
    torch.testing.assert_close(got.cpu(), torch.log_softmax(x, -1), atol=2e-5, rtol=0)
    one = log_softmax(x[rows - 1 : rows].cuda(), dim=-1)
    assert_bitwise(one, got[rows - 1 : rows], "log_softmax single row")
    with pytest.raises(ValueError):
        log_softmax(x.cuda(), dim=0)


def test_log_softmax_3d_and_bf16():
    x = _gen((2, 3, 500), 11)
    got = log_softmax(x.cuda(), dim=-1).cpu()
    torch.testing.assert_close(got, torch.log_softmax(x, -1), atol=2e-5, rtol=0)
    xb = x.to(torch.bfloat16)
    gb = log_softmax(xb.cuda(), dim=2).cpu()
    assert gb.dtype == torch.bfloat16
    torch.testing.assert_close(gb.float(), torch.log_softmax(xb.float(), -1), atol=6e-2, rtol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_log_softmax_and_logprobs_on_ragged_and_unaligned_rows(dtype):
    # rows that start at any element offset (column slices of a wider tensor) and lengths that are no multiple of
    # the 4-element vectors: the vector and the element-wise form of the loads must give the same bits
    wide = _gen((9, 9000), 21, dtype, scale=2.5).cuda()
    g = torch.Generator().manual_seed(22)
    for n in (8192, 8190, 4097, 4099, 5, 3):
        labels = torch.randint(0, n, (9,), generator=g).cuda()
        base = wide[:, :n].contiguous()
        want_ls = ops.log_softmax(base, -1)
        want_lp, want_tok = ops.logprobs(base, None, return_tokens=True)
        want_lab = ops.logprobs(base, labels)
        if dtype == torch.float32:
            torch.testing.assert_close(want_ls.cpu(), torch.log_softmax(base.cpu(), -1), atol=2e-5, rtol=0)
        for off in (1, 2, 3, 4):
            view = wide[:, off : off + n]
            shifted = wide.clone()
            shifted[:, off : off + n] = wide[:, :n]
            view = shifted[:, off : off + n]  # same values as `base`, rows starting `off` elements into the pitch
            assert_bitwise(ops.log_softmax(view, -1), want_ls, f"log_softmax n={n} offset {off}")
            lp, tok = ops.logprobs(view, None, return_tokens=True)
            assert_bitwise(lp, want_lp, f"greedy logprob n={n} offset {off}")
            assert torch.equal(tok, want_tok)
            assert_bitwise(ops.logprobs(view, labels), want_lab, f"label logprob n={n} offset {off}")


@pytest.mark.parametrize("vocab", [1000, 151936])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_logprobs_value_and_permutation_invariance(vocab, dtype):
    rows = 33
    logits = _gen((rows, vocab), 12, dtype, scale=2.0)
    g = torch.Generator().manual_seed(13)
    labels = torch.randint(0, vocab, (rows,), generator=g)
    got = logprobs_from_logits_flash_attn(logits.cuda(), labels.cuda())
    assert got.dtype == torch.float32 and got.shape == labels.shape
    ref = O.logprobs_ref(logits, labels)
    torch.testing.assert_close(got.cpu(), ref, atol=2e-5, rtol=0)  # stated bar is 2e-2
    perm = torch.randperm(rows, generator=g)
    got_p = logprobs_from_logits_flash_attn(logits[perm].cuda(), labels[perm].cuda())
    assert_bitwise(got_p, got[perm.cuda()], "logprobs under row permutation")
    one = logprobs_from_logits_flash_attn(logits[5:6].cuda(), labels[5:6].cuda())
    assert_bitwise(one, got[5:6], "logprobs single row")


def test_greedy_token_is_first_argmax():
    logits = _gen((17, 5000), 14)
    logits[3, 100] = logits[3, 4000] = 50.0  # tie: the lower index wins
    lp, tok = ops.logprobs(logits.cuda(), None, return_tokens=True)
    ref_tok = torch.tensor([int(torch.nonzero(r == r.max())[0]) for r in logits])
    assert torch.equal(tok.cpu(), ref_tok)
    torch.testing.assert_close(lp.cpu(), O.logprobs_ref(logits, ref_tok), atol=2e-5, rtol=0)


@pytest.mark.parametrize("rows,n,dtype", [(5, 1000, torch.bfloat16), (64, 151936, torch.bfloat16), (300, 4097, torch.float32),
                                         (3, 77, torch.float16)])
def test_logprobs_backward_matches_autograd_of_log_softmax(rows, n, dtype):
    # logprobs_from_logits_flash_attn under autograd: forward = the inference kernel's bits, backward = d_out (onehot - softmax)
    # against autograd through an fp32 log_softmax; the in-place form writes the same gradient into the logits
    from vexact_amd.batch_invariant_ops.standalone_logprobs import logprobs_from_logits_flash_attn
    g = torch.Generator().manual_seed(rows + n)
    logits = (3.0 * torch.randn(rows, n, generator=g)).to(dtype).cuda()
    labels = torch.randint(0, n, (rows,), generator=g).cuda()
    d_out = torch.randn(rows, generator=g).cuda()
    plain = logprobs_from_logits_flash_attn(logits, labels)
    x = logits.clone().requires_grad_()
    lp = logprobs_from_logits_flash_attn(x, labels)
    assert_bitwise(lp.detach(), plain, "forward under autograd")
    lp.backward(d_out)
    ref_x = logits.float().clone().requires_grad_()
    torch.log_softmax(ref_x, -1).gather(-1, labels[:, None])[:, 0].backward(d_out)
    want = ref_x.grad.to(dtype)
    err = (x.grad.float() - want.float()).abs()
    tol = 1e-5 if dtype == torch.float32 else 2.0 ** -7
    assert float((err / (want.float().abs() + 1e-3)).max()) <= tol, f"gradient: worst relative error {float((err / (want.float().abs() + 1e-3)).max()):.3g}"
    y = logits.clone().requires_grad_()
    z = y.clone()                                 # a non-leaf whose memory the in-place backward may take
    logprobs_from_logits_flash_attn(z, labels, inplace_backward=True).backward(d_out)
    assert_bitwise(y.grad, x.grad, "in-place backward")


@pytest.mark.parametrize("rows,n,dtype", [(37, 2048, torch.bfloat16), (1000, 128, torch.bfloat16), (5, 8192, torch.bfloat16),
                                         (3000, 256, torch.float16), (1, 64, torch.bfloat16), (70000, 128, torch.bfloat16)])
def test_rms_norm_backward_matches_autograd(rows, n, dtype):
    # vx_rms_norm_bwd against autograd through the fp32 formula of the HuggingFace forward (both roundings); deterministic
    g = torch.Generator().manual_seed(rows + n)
    x = torch.randn(rows, n, generator=g).to(dtype).cuda()
    w = (1.0 + 0.2 * torch.randn(n, generator=g)).to(dtype).cuda()
    dy = torch.randn(rows, n, generator=g).to(dtype).cuda()
    d_x, d_w = ops.rms_norm_backward(x, w, dy, 1e-6, hf_two_rounding=True)
    xr, wr = x.float().requires_grad_(), w.float().requires_grad_()
    h = xr * torch.rsqrt(xr.pow(2).mean(-1, keepdim=True) + 1e-6)
    (wr * h).backward(dy.float())
    for name, got, want in (("input", d_x, xr.grad), ("weight", d_w, wr.grad)):
        err, scale = (got.float() - want).abs(), float(want.abs().max())
        assert float(err.max()) <= 2.0 ** -6 * scale, f"{name} gradient: max err {float(err.max()):.4g} vs scale {scale:.4g}"
    again = ops.rms_norm_backward(x, w, dy, 1e-6, hf_two_rounding=True)
    assert_bitwise(again[0], d_x, "second launch, input gradient")
    assert_bitwise(again[1], d_w, "second launch, weight gradient")
    # a row's input gradient does not depend on the other rows
    one = ops.rms_norm_backward(x[rows // 2: rows // 2 + 1].contiguous(), w, dy[rows // 2: rows // 2 + 1].contiguous(), 1e-6,
                                hf_two_rounding=True)
    assert_bitwise(one[0], d_x[rows // 2: rows // 2 + 1], "row alone")


@pytest.mark.parametrize("shape,dtype", [((37, 2048), torch.bfloat16), ((2, 50, 128), torch.float16), ((9, 100), torch.bfloat16),
                                         ((4, 64), torch.float32)])
def test_batch_invariant_rms_norm_backward_matches_autograd(shape, dtype):
    # BatchInvariantRMSNormFunction.backward (the reference's: batch_invariant_ops.py:701-725) on vx_rms_norm_bwd in its
    # one-rounding form; rows the kernel does not take (fp32, a length that is not a multiple of 8) use tensor operations
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(shape, generator=g).to(dtype).cuda().requires_grad_()
    w = (1.0 + 0.2 * torch.randn(shape[-1], generator=g)).to(dtype).cuda().requires_grad_()
    dy = torch.randn(shape, generator=g).to(dtype).cuda()
    y = batch_invariant_rms_norm(x, w, 1e-6)
    y.backward(dy)
    xr, wr = x.detach().float().requires_grad_(), w.detach().float().requires_grad_()
    (xr * torch.rsqrt(xr.pow(2).mean(-1, keepdim=True) + 1e-6) * wr).backward(dy.float())
    assert x.grad.dtype == dtype and w.grad.dtype == dtype and x.grad.shape == x.shape and w.grad.shape == w.shape
    for name, got, want in (("input", x.grad, xr.grad), ("weight", w.grad, wr.grad)):
        err, scale = (got.float() - want).abs(), float(want.abs().max())
        assert float(err.max()) <= 2.0 ** -6 * scale, f"{name} gradient: max err {float(err.max()):.4g} vs scale {scale:.4g}"
