"""Comparators shared by the tests."""

import torch


def bits(t: torch.Tensor) -> torch.Tensor:
    """Raw bit pattern as integers (for exact comparisons that also distinguish -0 / NaN payloads)."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16)
    if t.dtype == torch.float32:
        return t.view(torch.int32)
    return t


def differing_bits(a: torch.Tensor, b: torch.Tensor) -> int:
    """Number of elements whose bit patterns differ."""
    assert a.shape == b.shape and a.dtype == b.dtype, (a.shape, b.shape, a.dtype, b.dtype)
    return int((bits(a) != bits(b)).sum())


def assert_bitwise(a, b, what=""):
    n = differing_bits(a, b)
    assert n == 0, f"{what}: {n} of {a.numel()} elements differ in bits"


def bf16_ulp_distance(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in bf16 units-in-the-last-place between two bf16 tensors."""
    def key(t):
        i = t.detach().cpu().contiguous().view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)
    return (key(a) - key(b)).abs()


def assert_bf16_close(a, b, max_ulp=2, atol_frac=1e-4, what=""):
    """Every element within ``max_ulp`` bf16 ulps, or within ``atol_frac * max|b|`` absolutely (the
    latter covers outputs that are small through cancellation, where fp32 accumulation-order noise
    exceeds the element's own ulp)."""
    a, b = a.detach().cpu(), b.detach().cpu()
    assert a.shape == b.shape, (a.shape, b.shape)
    ulp = bf16_ulp_distance(a, b)
    absd = (a.float() - b.float()).abs()
    atol = atol_frac * float(b.float().abs().max()) if b.numel() else 0.0
    bad = (ulp > max_ulp) & (absd > atol)
    assert not bool(bad.any()), (
        f"{what}: {int(bad.sum())} of {a.numel()} elements beyond {max_ulp} ulp "
        f"(worst {int(ulp.max())} ulp, |d|max {float(absd.max()):.3e}, atol {atol:.3e})"
    )


def ulp_histogram(a: torch.Tensor, b: torch.Tensor, what: str = "") -> dict:
    """Share of elements at 0 / 1 / 2 / more bf16 ulps from the reference, with no absolute floor; printed so
    that the tolerance a test meets is a measured one."""
    ulp = bf16_ulp_distance(a, b)
    n = max(1, ulp.numel())
    h = {"0": float((ulp == 0).sum()) / n, "1": float((ulp == 1).sum()) / n, "2": float((ulp == 2).sum()) / n,
         ">2": float((ulp > 2).sum()) / n, "worst": int(ulp.max()) if ulp.numel() else 0}
    print(f"[ulp] {what}: 0 ulp {h['0']:.4%}, 1 ulp {h['1']:.4%}, 2 ulp {h['2']:.4%}, >2 ulp {h['>2']:.4%} "
          f"(worst {h['worst']}) of {ulp.numel()} elements", flush=True)
    return h
