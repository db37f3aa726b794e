"""Torch-tensor front end of the C ABI: argument validation, output allocation, launches.

Every function here takes and returns ``torch`` tensors that live on the GPU and launches on
``torch.cuda.current_stream()``. Nothing falls back to PyTorch arithmetic: if the HIP library is
missing the call raises.
"""

from __future__ import annotations

import ctypes
import threading
from typing import Optional

import torch

from . import _lib

_DT = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need_gpu(name: str, t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must be a CUDA tensor")


_EMPTY_LOCK = threading.Lock()


def _empty(*size, **kw) -> torch.Tensor:
    """``torch.empty`` for a tensor that the kernel about to be launched writes completely. Under
    ``torch.use_deterministic_algorithms(True)`` (which ``enable_batch_invariant_mode`` turns on, as the
    reference's does) ``torch.empty`` fills what it returns with NaN, one more kernel in front of every op here
    (about 3 us each, some twenty per decoder layer); that fill is skipped for these tensors, whose every
    element is overwritten anyway. Attention outputs keep it: rows of a sequence without any key stay unwritten.
    The switch is a process-wide flag of torch: the lock keeps two threads of this package from restoring it in
    the wrong order, and the previous value (not ``True``) is what comes back. A ``torch.empty`` that another
    thread's own code issues inside that window still loses its fill; the reference runs one generation thread per
    process (vexact/worker/worker.py:48), which is the arrangement this is meant for."""
    det = torch.utils.deterministic
    if torch.are_deterministic_algorithms_enabled() and det.fill_uninitialized_memory:
        with _EMPTY_LOCK:
            previous = det.fill_uninitialized_memory
            det.fill_uninitialized_memory = False
            try:
                return torch.empty(*size, **kw)
            finally:
                det.fill_uninitialized_memory = previous
    return torch.empty(*size, **kw)


def _empty_like(t: torch.Tensor) -> torch.Tensor:
    return _empty(t.shape, dtype=t.dtype, device=t.device)


def _workspace(nbytes: int, device) -> torch.Tensor:
    return _empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)


# ----------------------------------------------------------------------------- row ops


def mean_dim(x: torch.Tensor, dim: int, keepdim: bool = False, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    _need_gpu("input", x)
    assert -x.ndim <= dim < x.ndim, f"Invalid dimension {dim} for tensor with {x.ndim} dimensions"
    if dim < 0:
        dim += x.ndim
    if dtype is None:
        dtype = torch.float32 if x.dtype in (torch.int8, torch.int16, torch.int32, torch.int64) else x.dtype
    if x.dtype != dtype:
        x = x.to(dtype)
    if dtype not in _DT:
        raise ValueError(f"mean_dim: unsupported dtype {dtype}")
    shape = list(x.shape)
    M = 1
    for s in shape[:dim]:
        M *= s
    N = shape[dim]
    K = 1
    for s in shape[dim + 1 :]:
        K *= s
    out_shape = shape.copy()
    if keepdim:
        out_shape[dim] = 1
    else:
        out_shape = shape[:dim] + shape[dim + 1 :]
    out = _empty(out_shape, dtype=dtype, device=x.device)
    if M * K == 0:
        return out
    if N == 0:
        return out.fill_(float("nan"))
    x3 = x.reshape(M, N, K)
    _lib.check(
        _lib.load().vx_mean_dim(
            x3.data_ptr(), out.data_ptr(), _DT[dtype], M, N, K, x3.stride(0), x3.stride(1), x3.stride(2), K, 1, _stream()
        ),
        "vx_mean_dim",
    )
    return out


def rms_norm(
    x: torch.Tensor,
    weight: torch.Tensor,
    eps: float = 1e-6,
    *,
    hf_two_rounding: bool = False,
    residual: Optional[torch.Tensor] = None,
    sum_out: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """RMSNorm over the last dim. With ``residual`` the row becomes ``x + residual`` first (rounded
    to the storage dtype) and that sum is written to ``sum_out`` when given."""
    _need_gpu("input", x)
    if x.dtype not in _DT:
        raise ValueError(f"rms_norm: unsupported dtype {x.dtype}")
    n = x.shape[-1]
    x2 = x.reshape(-1, n)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    w = weight.contiguous()
    if w.dtype != x.dtype:
        w = w.to(x.dtype)
    assert w.numel() == n, "weight must have the size of the last dim"
    y = out if out is not None else _empty((x2.shape[0], n), dtype=x.dtype, device=x.device)
    y2 = y.reshape(-1, n)
    r2 = s2 = None
    if residual is not None:
        r2 = residual.reshape(-1, n)
        assert r2.dtype == x.dtype and r2.stride(-1) == 1 and r2.shape == x2.shape
        if sum_out is not None:
            s2 = sum_out.reshape(-1, n)
            assert s2.dtype == x.dtype and s2.stride(-1) == 1 and s2.shape == x2.shape
    _lib.check(
        _lib.load().vx_rms_norm(
            x2.data_ptr(), _ptr(r2), w.data_ptr(), y2.data_ptr(), _ptr(s2), _DT[x.dtype], x2.shape[0], n,
            x2.stride(0), r2.stride(0) if r2 is not None else 0, y2.stride(0),
            s2.stride(0) if s2 is not None else 0, float(eps), 1 if hf_two_rounding else 0, _stream(),
        ),
        "vx_rms_norm",
    )
    return y.reshape(x.shape) if out is None else out


def rms_norm_backward(x: torch.Tensor, weight: torch.Tensor, d_y: torch.Tensor, eps: float = 1e-6, *,
                      hf_two_rounding: bool = False):
    """``(d_x, d_weight)`` of ``rms_norm(x, weight, eps)`` (no residual) for bf16 / fp16 rows of at most 8192 entries
    (a multiple of 8), in two launches."""
    _need_gpu("input", x)
    n = x.shape[-1]
    assert x.dtype in (torch.bfloat16, torch.float16) and n % 8 == 0 and n <= 8192 and d_y.shape == x.shape
    x2 = x.reshape(-1, n)
    g2 = d_y.reshape(-1, n).to(x.dtype)
    if x2.stride(-1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    if g2.stride(-1) != 1 or g2.stride(0) % 8 or g2.data_ptr() % 16:
        g2 = g2.contiguous()
    w = weight.to(x.dtype).contiguous()
    rows = x2.shape[0]
    d_x = _empty((rows, n), dtype=x.dtype, device=x.device)
    d_w = _empty((n,), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    ws = _workspace(lib.vx_rms_norm_bwd_workspace_bytes(rows, n), x.device)
    _lib.check(
        lib.vx_rms_norm_bwd(x2.data_ptr(), w.data_ptr(), g2.data_ptr(), d_x.data_ptr(), d_w.data_ptr(), _DT[x.dtype], rows, n,
                            x2.stride(0), g2.stride(0), d_x.stride(0), float(eps), 1 if hf_two_rounding else 0,
                            ws.data_ptr(), ws.numel(), _stream()),
        "vx_rms_norm_bwd",
    )
    return d_x.reshape(x.shape), d_w


def log_softmax(x: torch.Tensor, dim: int = -1) -> torch.Tensor:
    if dim != -1 and dim != x.ndim - 1:
        raise ValueError("This implementation only supports log_softmax along the last dimension")
    _need_gpu("input", x)
    if x.dtype not in _DT:
        raise ValueError(f"log_softmax: unsupported dtype {x.dtype}")
    shape = x.shape
    x2 = x.reshape(-1, shape[-1]).contiguous()
    rows, n = x2.shape
    y = _empty_like(x2)
    if rows == 0 or n == 0:
        return y.reshape(shape)
    lib = _lib.load()
    step = 65535  # grid.y limit
    for r0 in range(0, rows, step):
        r = min(step, rows - r0)
        ws = _workspace(lib.vx_log_softmax_workspace_bytes(r, n), x.device)
        _lib.check(
            lib.vx_log_softmax(
                x2[r0:].data_ptr(), y[r0:].data_ptr(), _DT[x.dtype], r, n, x2.stride(0), y.stride(0),
                ws.data_ptr(), ws.numel(), _stream(),
            ),
            "vx_log_softmax",
        )
    return y.reshape(shape)


def logprobs(
    logits: torch.Tensor, labels: Optional[torch.Tensor], *, return_tokens: bool = False
):
    """Per-row ``logits[i, labels[i]] - logsumexp(logits[i])`` in fp32. ``labels=None`` scores the
    greedy (first-argmax) token and can return it."""
    _need_gpu("logits", logits)
    if logits.dtype not in _DT:
        raise ValueError(f"logprobs: unsupported dtype {logits.dtype}")
    x2 = logits.reshape(-1, logits.shape[-1])
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    rows, n = x2.shape
    out = _empty(rows, dtype=torch.float32, device=logits.device)
    toks = _empty(rows, dtype=torch.int64, device=logits.device) if (return_tokens or labels is None) else None
    lab = None
    if labels is not None:
        lab = labels.reshape(-1)
        if lab.dtype != torch.int64:
            lab = lab.to(torch.int64)
        lab = lab.contiguous()
        assert lab.numel() == rows, "labels must have one entry per row"
    if rows == 0:
        return (out, toks) if return_tokens else out
    lib = _lib.load()
    step = 65535
    for r0 in range(0, rows, step):
        r = min(step, rows - r0)
        ws = _workspace(lib.vx_log_softmax_workspace_bytes(r, n), logits.device)
        _lib.check(
            lib.vx_logprobs(
                x2[r0:].data_ptr(), _ptr(lab[r0:]) if lab is not None else None, out[r0:].data_ptr(),
                _ptr(toks[r0:]) if toks is not None else None, _DT[logits.dtype], r, n, x2.stride(0),
                ws.data_ptr(), ws.numel(), _stream(),
            ),
            "vx_logprobs",
        )
    return (out, toks) if return_tokens else out


def logprobs_backward(logits: torch.Tensor, labels: torch.Tensor, out: torch.Tensor, d_out: torch.Tensor,
                      inplace: bool = False) -> torch.Tensor:
    """Gradient of ``logprobs(logits, labels)`` with respect to ``logits [rows, n]`` given the forward's ``out`` and
    the incoming ``d_out`` (both fp32 ``[rows]``); ``inplace`` writes it over the logits."""
    _need_gpu("logits", logits)
    assert logits.dim() == 2 and logits.stride(1) == 1 and logits.dtype in _DT
    rows, n = logits.shape
    lab = labels.reshape(-1).to(torch.int64).contiguous()
    o, g = out.reshape(-1).float().contiguous(), d_out.reshape(-1).float().contiguous()
    assert lab.numel() == rows and o.numel() == rows and g.numel() == rows
    d = logits if inplace else _empty_like(logits)
    lib = _lib.load()
    for r0 in range(0, rows, 65535):
        r = min(65535, rows - r0)
        _lib.check(
            lib.vx_logprobs_bwd(logits[r0:].data_ptr(), lab[r0:].data_ptr(), o[r0:].data_ptr(), g[r0:].data_ptr(),
                                d[r0:].data_ptr(), _DT[logits.dtype], r, n, logits.stride(0), d.stride(0), _stream()),
            "vx_logprobs_bwd",
        )
    return d


def sample_tokens(
    logits: torch.Tensor, temperature: float, top_k: Optional[int], top_p: float, seeds: torch.Tensor,
    positions: torch.Tensor, out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """One sampled token per row of ``logits`` [B, V] (bf16 or fp32): temperature, top-k, top-p and a
    Philox-seeded exponential race in one kernel. ``seeds`` / ``positions`` are int64 [B] on the device;
    a row's token depends only on (its logits, its seed, its position)."""
    _need_gpu("logits", logits)
    if logits.dim() != 2 or logits.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"sample_tokens: need [B, V] bf16 or fp32 logits, got {tuple(logits.shape)} {logits.dtype}")
    if logits.stride(1) != 1:
        logits = logits.contiguous()
    B, V = logits.shape
    if not (temperature > 0 and top_p > 0):
        raise ValueError("sample_tokens: temperature and top_p must be positive (greedy decoding is logprobs(labels=None))")
    for name, t in (("seeds", seeds), ("positions", positions)):
        if t.dtype != torch.int64 or t.numel() != B or not t.is_contiguous() or t.device != logits.device:
            raise ValueError(f"sample_tokens: {name} must be a contiguous int64 [B] tensor on the logits' device")
    if out is None:
        out = _empty(B, dtype=torch.int64, device=logits.device)
    _lib.check(
        _lib.load().vx_sample_tokens(
            logits.data_ptr(), 0 if logits.dtype == torch.bfloat16 else 1, logits.stride(0), B, V, float(temperature),
            int(top_k) if top_k is not None else 0, float(top_p), seeds.data_ptr(), positions.data_ptr(), out.data_ptr(),
            _stream(),
        ),
        "vx_sample_tokens",
    )
    return out


# ----------------------------------------------------------------------------- GEMM


def _fast_ok(x: torch.Tensor, w_nk: torch.Tensor) -> bool:
    K = x.shape[1]
    return (
        x.dtype == torch.bfloat16
        and w_nk.dtype == torch.bfloat16
        and x.stride(1) == 1
        and w_nk.stride(1) == 1
        and K % 8 == 0
        and x.stride(0) % 8 == 0
        and w_nk.stride(0) % 8 == 0
        and x.data_ptr() % 16 == 0
        and w_nk.data_ptr() % 16 == 0
    )


def gemm_nt(
    x: torch.Tensor, w_nk: torch.Tensor, bias: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None
) -> torch.Tensor:
    """``x[M,K] @ w_nk[N,K].T (+ bias)`` in bf16 on the MFMA path (raises if the layout does not fit)."""
    M, K = x.shape
    N = w_nk.shape[0]
    c = out if out is not None else _empty((M, N), dtype=x.dtype, device=x.device)
    assert c.stride(1) == 1
    _lib.check(
        _lib.load().vx_gemm_bf16_nt(
            x.data_ptr(), w_nk.data_ptr(), _ptr(bias), c.data_ptr(), M, N, K, x.stride(0), w_nk.stride(0),
            c.stride(0), _stream(),
        ),
        "vx_gemm_bf16_nt",
    )
    return c


def gemm_nt_variant(x: torch.Tensor, w_nk: torch.Tensor, kind: int, mt: int = 1, bias=None) -> torch.Tensor:
    M, K = x.shape
    N = w_nk.shape[0]
    c = _empty((M, N), dtype=x.dtype, device=x.device)
    _lib.check(
        _lib.load().vx_gemm_bf16_nt_variant(
            x.data_ptr(), w_nk.data_ptr(), _ptr(bias), c.data_ptr(), M, N, K, x.stride(0), w_nk.stride(0),
            c.stride(0), kind, mt, _stream(),
        ),
        "vx_gemm_bf16_nt_variant",
    )
    return c


def gemm_swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, out: Optional[torch.Tensor] = None,
                kind: int = -1, mt: int = 1) -> torch.Tensor:
    """``silu(x @ w_gate.T) * (x @ w_up.T)`` with every bf16 rounding of the unfused chain, in one
    kernel. ``x`` [M, K], ``w_gate`` / ``w_up`` [N, K] bf16 with the same row pitch."""
    _need_gpu("x", x)
    if not (_fast_ok(x, w_gate) and _fast_ok(x, w_up)) or w_gate.shape != w_up.shape or w_gate.stride(0) != w_up.stride(0):
        raise ValueError("gemm_swiglu: need K-contiguous, 16-byte aligned bf16 operands; gate and up of one shape and pitch")
    M, K = x.shape
    N = w_gate.shape[0]
    if out is None:
        out = _empty(M, N, dtype=torch.bfloat16, device=x.device)
    _lib.check(
        _lib.load().vx_gemm_swiglu_bf16_nt(x.data_ptr(), w_gate.data_ptr(), w_up.data_ptr(), out.data_ptr(), M, N, K,
                                           x.stride(0), w_gate.stride(0), out.stride(0), kind, mt, _stream()),
        "vx_gemm_swiglu_bf16_nt",
    )
    return out


def swiglu_mlp(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """Dense SwiGLU MLP ``down_proj(act_fn(gate_proj(x)) * up_proj(x))`` in two kernels."""
    return gemm_nt(gemm_swiglu(x, w_gate, w_up), w_down)


_ROW_SPANS: dict = {}


def _row_span(rows: int, device) -> torch.Tensor:
    """``[0, rows]`` as an int32 device tensor (the row offsets of a single group), made once per size."""
    key = (int(rows), str(device))
    t = _ROW_SPANS.get(key)
    if t is None:
        if len(_ROW_SPANS) > 256:
            _ROW_SPANS.clear()
        t = torch.tensor([0, int(rows)], dtype=torch.int32, device=device)
        _ROW_SPANS[key] = t
    return t


_ONE_GROUP_TILES: dict = {}


def _one_group_tiles(rows: int, device):
    """The 256-row tile table of a single group holding ``rows`` rows, in the form ``moe_gemm_nn`` reads (made
    once per size)."""
    from types import SimpleNamespace

    key = (int(rows), str(device))
    r = _ONE_GROUP_TILES.get(key)
    if r is None:
        if len(_ONE_GROUP_TILES) > 64:
            _ONE_GROUP_TILES.clear()
        n = (rows + 255) // 256
        row0 = torch.arange(0, n * 256, 256, dtype=torch.int32, device=device)
        r = SimpleNamespace(T=rows, k=1, bm=256, max_tiles=n, tile_group=torch.zeros(n, dtype=torch.int32, device=device),
                            tile_row0=row0, tile_rows=torch.clamp(rows - row0, max=256).to(torch.int32))
        _ONE_GROUP_TILES[key] = r
    return r


def matmul(a: torch.Tensor, b: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``a[M,K] @ b[K,N] (+ bias[N])`` with the dtype of ``a``; any strides.

    bf16 operands go through the MFMA kernels: directly when ``b`` is a transposed view of an
    ``[N, K]`` row-major weight (the ``nn.Linear`` case), after packing ``b`` otherwise. fp16 and fp32
    have an MFMA kernel of their own (true fp32 products for fp32). Unaligned bf16 layouts use the
    generic one-thread-per-output kernel. Large bf16 products whose ``b`` is row-major ``[K, N]`` (data gradients)
    or whose ``a`` is a transposed view as well (weight gradients) run on the grouped backward kernels with a
    single group instead of going through transposed copies. Every bf16 MFMA kernel gives the same bits for the
    same row, so which one runs (it may depend on M) changes no result.
    """
    assert a.ndim == 2 and b.ndim == 2, "matmul expects 2-D operands"
    assert a.shape[1] == b.shape[0], "Incompatible dimensions"
    assert a.dtype == b.dtype, "Incompatible dtypes"
    assert bias is None or bias.dim() == 1, "Currently assuming bias is 1D, let Horace know if you run into this"
    _need_gpu("a", a)
    if a.dtype not in _DT:
        raise ValueError(f"matmul: unsupported dtype {a.dtype}")
    M, K = a.shape
    N = b.shape[1]
    if bias is not None:
        bias = bias.to(a.dtype).contiguous()
    c = _empty((M, N), dtype=a.dtype, device=a.device)
    if M == 0 or N == 0:
        return c
    if K == 0:
        c.zero_()
        if bias is not None:
            c += bias
        return c
    lib = _lib.load()
    if (a.dtype == torch.bfloat16 and bias is None and a.stride(0) == 1 and b.stride(1) == 1 and M % 8 == 0 and N % 8 == 0
            and a.stride(1) % 8 == 0 and b.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and b.data_ptr() % 16 == 0
            and ((M + 255) // 256) * ((N + 255) // 256) >= 96 and not torch.cuda.is_current_stream_capturing()):
        # a is the transposed view of a row-major [K, M] tensor and b is row-major [K, N] (a linear layer's weight
        # gradient, d_y^T x): the contraction index is the slow index of both, which the grouped weight-gradient
        # kernel reads as it lies (one group holding every row) instead of two transposed copies; same MFMA chain per
        # output element as the other kernels. Only with enough 256 x 256 output tiles to occupy the chip.
        return moe_gemm_tn(a.t(), b, _row_span(K, a.device), 1, out=c.view(1, M, N)).view(M, N)
    if (a.dtype == torch.bfloat16 and bias is None and a.stride(1) == 1 and b.stride(1) == 1 and b.stride(0) != 1
            and M >= 1024 and K % 64 == 0 and N % 8 == 0 and a.stride(0) % 8 == 0 and b.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and b.data_ptr() % 16 == 0 and (M * a.stride(0) + K) * 2 < (1 << 32)
            and (64 * b.stride(0) + N) * 2 < (1 << 32) and not torch.cuda.is_current_stream_capturing()):
        # b is row-major [K, N] (a linear layer's data gradient, d_y w): the grouped data-gradient kernel reads it as
        # it lies, with all rows in one group, instead of a transposed copy of the weight in front of an NT kernel;
        # same MFMA chain per output element
        return moe_gemm_nn(a, b.unsqueeze(0), _one_group_tiles(M, a.device), out=c)
    if a.dtype == torch.bfloat16 and K % 8 == 0:
        w_nk = b.t()  # [N, K] view
        x = a
        if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.data_ptr() % 16 != 0:
            x = a.contiguous()
        if w_nk.stride(1) != 1 or w_nk.stride(0) % 8 != 0 or w_nk.data_ptr() % 16 != 0:
            # pack b[K, N] (any strides) into an [N, K] row-major buffer
            bc = b if b.stride(1) == 1 else b.contiguous()
            packed = _empty((N, K), dtype=b.dtype, device=b.device)
            _lib.check(
                lib.vx_transpose_bf16(bc.data_ptr(), packed.data_ptr(), K, N, bc.stride(0), K, _stream()),
                "vx_transpose_bf16",
            )
            w_nk = packed
        if _fast_ok(x, w_nk):
            return gemm_nt(x, w_nk, bias, out=c)
    if a.dtype in (torch.float32, torch.float16):
        # matrix cores for these too: one kernel and tile shape for every M; operands made K-contiguous if needed
        x = a if a.stride(1) == 1 else a.contiguous()
        w_nk = b.t() if b.stride(0) == 1 else b.t().contiguous()
        _lib.check(
            lib.vx_gemm_nt_mfma(x.data_ptr(), w_nk.data_ptr(), _ptr(bias), c.data_ptr(), _DT[a.dtype], M, N, K,
                                x.stride(0), w_nk.stride(0), c.stride(0), _stream()),
            "vx_gemm_nt_mfma",
        )
        return c
    _lib.check(
        lib.vx_gemm_generic(
            a.data_ptr(), b.data_ptr(), _ptr(bias), c.data_ptr(), _DT[a.dtype], 1, M, N, K,
            0, a.stride(0), a.stride(1), 0, b.stride(0), b.stride(1), 0, c.stride(0), c.stride(1), _stream(),
        ),
        "vx_gemm_generic",
    )
    return c


def bmm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    assert a.ndim == 3 and b.ndim == 3, f"Expected 3D tensors, got {a.ndim}D and {b.ndim}D"
    B, M, K = a.shape
    _, K2, N = b.shape
    assert K == K2 and a.shape[0] == b.shape[0]
    _need_gpu("a", a)
    if a.dtype not in _DT or a.dtype != b.dtype:
        raise ValueError(f"bmm: unsupported dtypes {a.dtype}, {b.dtype}")
    c = _empty((B, M, N), dtype=a.dtype, device=a.device)
    if c.numel() == 0:
        return c
    lib = _lib.load()
    step = 65535
    for b0 in range(0, B, step):
        nb = min(step, B - b0)
        _lib.check(
            lib.vx_gemm_generic(
                a[b0:].data_ptr(), b[b0:].data_ptr(), None, c[b0:].data_ptr(), _DT[a.dtype], nb, M, N, K,
                a.stride(0), a.stride(1), a.stride(2), b.stride(0), b.stride(1), b.stride(2),
                c.stride(0), c.stride(1), c.stride(2), _stream(),
            ),
            "vx_gemm_generic",
        )
    return c


# ----------------------------------------------------------------------------- KV cache + attention


def store_kvcache(key, value, k_cache, v_cache, slot_mapping) -> None:
    assert slot_mapping.numel() == key.shape[0]
    strided = False
    for name, t, cache in (("key", key, k_cache), ("value", value, v_cache)):
        N, H, D = t.shape
        assert t.stride(-1) == 1
        assert t.stride(1) == D
        assert cache.dtype == t.dtype, f"{name} and its cache must share a dtype"
        if cache.dim() == 4 and cache.shape[2:] == (H, D) and cache.stride(3) == 1 and cache.stride(1) != H * D:
            strided = True  # a [blocks, page, heads, D] view of other memory (KVCacheStore(head_major=True))
        else:
            assert cache.stride(1) == H * D, f"Cache stride mismatch: expected stride(1)={H * D}, got {cache.stride(1)}"
    if slot_mapping.dtype != torch.int32:
        raise ValueError(f"slot_mapping must have dtype torch.int32, got {slot_mapping.dtype}")
    es = key.element_size()
    if strided:
        assert k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[1] == v_cache.shape[1]
        _lib.check(
            _lib.load().vx_store_kvcache_strided(
                key.data_ptr(), value.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(),
                key.shape[0], key.shape[1], key.stride(0) * es, value.stride(0) * es, key.shape[2] * es, value.shape[2] * es,
                k_cache.shape[1], k_cache.stride(0) * es, k_cache.stride(1) * es, k_cache.stride(2) * es,
                v_cache.stride(0) * es, v_cache.stride(1) * es, v_cache.stride(2) * es, _stream(),
            ),
            "vx_store_kvcache_strided",
        )
        return
    _lib.check(
        _lib.load().vx_store_kvcache(
            key.data_ptr(), value.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(),
            key.shape[0], key.stride(0) * es, value.stride(0) * es, key.shape[1] * key.shape[2] * es,
            value.shape[1] * value.shape[2] * es, _stream(),
        ),
        "vx_store_kvcache",
    )


def _attn_dtype_code(what: str, *tensors: torch.Tensor) -> int:
    """0 for bf16, 1 for fp16, 2 for fp32 (the C ABI's dtype code); every tensor must share it. fp32, which the
    reference's kernels also take (its own backward tests run in it), goes to a correctness path of one thread per
    output row with true fp32 products; the 16-bit types are the tuned ones."""
    codes = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}
    dt = tensors[0].dtype
    if dt not in codes or any(t.dtype != dt for t in tensors):
        raise ValueError(f"{what} supports bfloat16, float16 or float32 tensors of one dtype, got {[str(t.dtype) for t in tensors]}")
    return codes[dt]


def paged_attention(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    seqused_k: torch.Tensor,
    page_table: torch.Tensor,
    softmax_scale: float,
    max_seqlen_q: int = 0,
    out: Optional[torch.Tensor] = None,
    workspace: Optional[torch.Tensor] = None,
    decode_kernel: str = "auto",
    seq_order: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Causal paged attention. ``max_seqlen_q == 1`` selects the split-KV decode kernels; any other
    value the general kernel (identical bits per row). ``decode_kernel`` forces one of the two decode
    forms ("split": one wavefront per 256-key chunk plus a combine launch, "fused": chunks folded
    inside one workgroup per (sequence, kv head)); "auto" picks by batch size. Same bits either way.
    ``seq_order`` (int32 permutation of the sequences) is the order in which the decode workgroups take the
    sequences (in a general launch: those of the decode kernel that takes the sequences of one query row);
    longest first shortens the tail of a batch of mixed lengths."""
    T, Hq, Dk = q.shape
    Hkv, Dv = k_cache.shape[2], v_cache.shape[-1]
    o = out if out is not None else torch.empty((T, Hq, Dv), dtype=q.dtype, device=q.device)
    if T == 0:
        return o
    dtype = _attn_dtype_code("paged attention", q, k_cache, v_cache, o)
    if Dk > 256 or Dv > 256:
        raise ValueError(f"head_dim must be <= 256, got {Dk}")
    if q.stride(-1) != 1 or k_cache.stride(-1) != 1 or v_cache.stride(-1) != 1 or o.stride(-1) != 1:
        raise ValueError("q, k, v and out must be contiguous in the head dimension")
    lib = _lib.load()
    B = seqused_k.numel()
    page = k_cache.shape[1]
    max_pages = page_table.shape[1]
    mode = {"auto": 0, "split": 3, "fused": 4}[decode_kernel] if max_seqlen_q == 1 else 1
    ws = None
    if mode != 1:  # only the split decode form keeps chunk states in memory; the fused form needs none
        need = lib.vx_paged_attn_decode_workspace_needed(B, Hq, Hkv, Dv, max_pages * page, mode)
        if need > 0:
            ws = workspace if workspace is not None and workspace.numel() * workspace.element_size() >= need else _workspace(need, q.device)
    if seq_order is not None and (seq_order.dtype != torch.int32 or seq_order.numel() != B or not seq_order.is_contiguous()):
        raise ValueError("seq_order must be a contiguous int32 permutation of the sequences")
    _lib.check(
        lib.vx_attention_typed(
            q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), o.data_ptr(), None, _ptr(seq_order),
            cu_seqlens_q.data_ptr(), seqused_k.data_ptr(), None, page_table.data_ptr(), T, B, Hq, Hkv, Dk, Dv,
            q.stride(0), q.stride(1), k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
            v_cache.stride(0), v_cache.stride(1), v_cache.stride(2), o.stride(0), o.stride(1),
            page_table.stride(0), max_pages, page, float(softmax_scale), 1, mode, int(max_seqlen_q), dtype,
            _ptr(ws), ws.numel() * ws.element_size() if ws is not None else 0, _stream(),
        ),
        "vx_attention",
    )
    return o


def packed_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    softmax_scale: float,
    causal: bool,
    max_seqlen_q: int = 0,
    return_lse: bool = False,
):
    """Varlen attention on packed (non-paged) K/V ``[Tk, Hkv, D]``; same arithmetic as the paged path.
    ``return_lse`` also returns the rows' fp32 log-sum-exp ``[T, Hq]`` (what the backward needs)."""
    T, Hq, Dk = q.shape
    Hkv, Dv = k.shape[1], v.shape[-1]
    # zeros, as the reference allocates its packed output (triton_invariant_attention.py:733): the rows of a sequence
    # that has queries but no keys are written by no kernel (rows that merely see no key under the mask are: as 0)
    o = torch.zeros((T, Hq, Dv), dtype=q.dtype, device=q.device)
    lse = torch.empty((T, Hq), dtype=torch.float32, device=q.device) if return_lse else None
    if T == 0:
        return (o, lse) if return_lse else o
    dtype = _attn_dtype_code("attention", q, k, v)
    if Dk > 256 or Dv > 256:
        raise ValueError(f"head_dim must be <= 256, got {Dk}")
    if q.stride(-1) != 1 or k.stride(-1) != 1 or v.stride(-1) != 1:
        raise ValueError("q, k and v must be contiguous in the head dimension")
    B = cu_seqlens_q.numel() - 1
    _lib.check(
        _lib.load().vx_attention_typed(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), _ptr(lse), None, cu_seqlens_q.data_ptr(), None,
            cu_seqlens_k.data_ptr(), None, T, B, Hq, Hkv, Dk, Dv, q.stride(0), q.stride(1),
            0, k.stride(0), k.stride(1), 0, v.stride(0), v.stride(1), o.stride(0), o.stride(1),
            0, 0, 0, float(softmax_scale), 1 if causal else 0, 2, int(max_seqlen_q), dtype, None, 0, _stream(),
        ),
        "vx_attention",
    )
    return (o, lse) if return_lse else o


def packed_attention_backward(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, dout: torch.Tensor, lse: torch.Tensor,
    cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor, softmax_scale: float, max_seqlen_q: int, max_seqlen_k: int,
):
    """(dq, dk, dv) of causal ``packed_attention`` (bf16, fp16 or fp32, head sizes up to 256; shapes of q, k, v)."""
    for name, t in (("q", q), ("k", k), ("v", v), ("out", out), ("dout", dout)):
        _need_gpu(name, t)
        if t.dim() != 3 or t.stride(2) != 1:
            raise ValueError(f"attention backward: {name} must be [tokens, heads, dim] with a contiguous last dim")
    dtype = _attn_dtype_code("attention backward", q, k, v, out, dout)
    T, Hq, D = q.shape
    Tk, Hkv, Dv = v.shape
    if k.shape != (Tk, Hkv, D) or out.shape != (T, Hq, Dv) or dout.shape != (T, Hq, Dv):
        raise ValueError("attention backward: q / k and v / out / dout shapes do not match")
    if D > 256 or Dv > 256:
        raise ValueError(f"head_dim must be <= 256, got {D}")
    if lse.dtype != torch.float32 or lse.shape != (T, Hq) or not lse.is_contiguous():
        raise ValueError("attention backward: lse must be a contiguous fp32 [tokens, heads] tensor")
    dq, dk, dv = _empty_like(q), _empty_like(k), _empty_like(v)
    if T == 0 or Tk == 0:
        return dq.zero_(), dk.zero_(), dv.zero_()
    lib = _lib.load()
    ws = _workspace(lib.vx_attention_bwd_workspace_bytes(T, Hq), q.device)
    strides = (ctypes.c_int64 * 16)(*[s for t in (q, k, v, out, dout, dq, dk, dv) for s in (t.stride(0), t.stride(1))])
    _lib.check(
        lib.vx_attention_bwd_typed(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dout.data_ptr(), lse.data_ptr(), dq.data_ptr(),
            dk.data_ptr(), dv.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), T, Tk,
            cu_seqlens_q.numel() - 1, Hq, Hkv, D, Dv, strides, float(softmax_scale), int(max_seqlen_q), int(max_seqlen_k),
            dtype, ws.data_ptr(), ws.numel(), _stream(),
        ),
        "vx_attention_bwd",
    )
    return dq, dk, dv


# ----------------------------------------------------------------------------- MoE


def router_topk(
    logits: torch.Tensor, top_k: int, renorm: bool = True, out_dtype: torch.dtype = torch.bfloat16,
    index_dtype: torch.dtype = torch.int64,
):
    """softmax(fp32) -> top-k (ties: lower expert index first) -> renorm -> cast."""
    _need_gpu("logits", logits)
    T, E = logits.shape
    if logits.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("router logits must be float32 or bfloat16")
    if out_dtype not in (torch.float32, torch.bfloat16) or index_dtype not in (torch.int32, torch.int64):
        raise ValueError("unsupported router output dtypes")
    lg = logits if logits.stride(1) == 1 else logits.contiguous()
    w = _empty((T, top_k), dtype=out_dtype, device=logits.device)
    idx = _empty((T, top_k), dtype=index_dtype, device=logits.device)
    _lib.check(
        _lib.load().vx_router_topk(
            lg.data_ptr(), w.data_ptr(), idx.data_ptr(), T, E, top_k, lg.stride(0),
            int(lg.dtype == torch.bfloat16), int(out_dtype == torch.bfloat16), int(index_dtype == torch.int64),
            int(renorm), _stream(),
        ),
        "vx_router_topk",
    )
    return w, idx


def router_topk_backward(logits: torch.Tensor, selected: torch.Tensor, d_weights: torch.Tensor, renorm: bool = True) -> torch.Tensor:
    """Gradient of ``router_topk(logits, k, renorm)[0]`` with respect to ``logits [T, E]`` (E <= 512, k <= 64)."""
    _need_gpu("logits", logits)
    T, E = logits.shape
    k = selected.shape[1]
    assert logits.dtype in (torch.float32, torch.bfloat16) and selected.dtype == torch.int64 and selected.shape == (T, k)
    lg = logits if logits.stride(1) == 1 else logits.contiguous()
    dw = d_weights if d_weights.dtype in (torch.float32, torch.bfloat16) else d_weights.float()
    dw, sel = dw.contiguous(), selected.contiguous()
    out = _empty((T, E), dtype=logits.dtype, device=logits.device)
    _lib.check(
        _lib.load().vx_router_topk_bwd(lg.data_ptr(), sel.data_ptr(), dw.data_ptr(), out.data_ptr(), T, E, k, lg.stride(0),
                                       out.stride(0), int(lg.dtype == torch.bfloat16), int(dw.dtype == torch.bfloat16),
                                       int(renorm), _stream()),
        "vx_router_topk_bwd",
    )
    return out


def moe_tile_rows(num_tokens: int, wide_ok: bool = True, packed_only: bool = False, packed: bool = False,
                  top_k: int = 8, num_experts: int = 128) -> int:
    """Rows per expert tile (any choice gives the same bits), chosen from the average number of rows an expert
    receives, ``num_tokens * top_k / num_experts``: that, not the token count, decides how full a tile is. The
    crossovers were measured at 128 experts / top-8 and are stated below as token counts of that shape (16 tokens
    per average expert row); other shapes are mapped onto it.
    ``wide_ok``: both GEMM depths are multiples of 64, which the 256-row kernel needs.
    ``packed``: fragment-order weights are at hand; ``packed_only``: nothing else is, and the 128-row kernel does
    not read them. With fragment-order weights the 256-row kernel overtakes the streaming kernel early (128 experts,
    top-8, measured per block: 448 tokens 256 us on 32-row tiles against 269 on 64-row ones; 768 tokens 309 on 64-row
    tiles against 314 on 256-row ones; 1024 tokens 365 against 311; 1536 tokens 318 against 353 on the 128-row kernel)."""
    if int(num_tokens) <= 16:
        # an expert receives at most one row per token (a top-k's experts are distinct; duplicates just make more
        # tiles): one 16-row tile each, half the matrix instructions of a 32-row
        # tile (gate/up at 1 .. 16 tokens 2 us faster), and the form that a launch of a few tiles runs as one-wavefront
        # blocks (1 token 23.8 -> 18.2 us, 4 tokens 46.5 -> 41.0 us)
        return 16
    eq = (int(num_tokens) * max(1, int(top_k)) * 16) // max(1, int(num_experts))  # token count of the measured shape
    if packed or packed_only:
        if eq <= 448:
            return 32
        if eq <= 832 or not wide_ok:
            return 64
        return 256
    # [E, N, K] tensors only (same block): 384 tokens 269 us on 32-row tiles against 297 on 64-row ones, 512 tokens
    # 311 / 306, 768 tokens 343 on 64-row tiles against 326 on 128-row ones, 1024 tokens 410 / 332
    if eq <= 448:
        return 32
    if eq <= 704:
        return 64
    if eq < 2048 or not wide_ok:
        return 128
    return 256


class MoeRouting:
    """Device-side routing integers produced by ``vx_moe_route``."""

    __slots__ = ("splits", "cu", "scatter_index", "sorted_token", "sorted_flat", "tile_group", "tile_row0",
                 "tile_rows", "max_tiles", "bm", "T", "k", "E")


def moe_route(selected_experts: torch.Tensor, num_experts: int, bm: Optional[int] = None, buffers=None,
              chunked: bool = True) -> MoeRouting:
    """Routing integers of ``selected_experts [T, k]``. From 3072 entries on the work is spread over many
    workgroups (needs a small workspace); ``chunked=False`` keeps the one-workgroup kernel (same integers)."""
    _need_gpu("selected_experts", selected_experts)
    assert selected_experts.dtype in (torch.int32, torch.int64)
    idx = selected_experts.contiguous()
    T, k = idx.shape
    bm = bm or moe_tile_rows(T, top_k=k, num_experts=num_experts)
    lib = _lib.load()
    max_tiles = lib.vx_moe_max_tiles(T * k, num_experts, bm)
    dev = idx.device
    r = MoeRouting()
    r.T, r.k, r.E, r.bm, r.max_tiles = T, k, num_experts, bm, max_tiles
    n = T * k
    if buffers is None:
        ints = _empty(num_experts + (num_experts + 1) + 3 * n + 3 * max_tiles, dtype=torch.int32, device=dev)
    else:
        ints = buffers
    o = 0
    r.splits = ints[o : o + num_experts]; o += num_experts
    r.cu = ints[o : o + num_experts + 1]; o += num_experts + 1
    r.scatter_index = ints[o : o + n].view(T, k); o += n
    r.sorted_token = ints[o : o + n]; o += n
    r.sorted_flat = ints[o : o + n]; o += n
    r.tile_group = ints[o : o + max_tiles]; o += max_tiles
    r.tile_row0 = ints[o : o + max_tiles]; o += max_tiles
    r.tile_rows = ints[o : o + max_tiles]; o += max_tiles
    need = lib.vx_moe_route_workspace_bytes(n, num_experts) if chunked else 0
    ws = _workspace(need, dev) if need > 0 else None
    _lib.check(
        lib.vx_moe_route_ws(
            idx.data_ptr(), int(idx.dtype == torch.int64), T, k, num_experts, bm, r.splits.data_ptr(),
            r.cu.data_ptr(), r.scatter_index.data_ptr(), r.sorted_token.data_ptr(), r.sorted_flat.data_ptr(),
            r.tile_group.data_ptr(), r.tile_row0.data_ptr(), r.tile_rows.data_ptr(), max_tiles, _ptr(ws),
            ws.numel() * ws.element_size() if ws is not None else 0, _stream(),
        ),
        "vx_moe_route",
    )
    return r


def moe_gemm(
    x: torch.Tensor, w: torch.Tensor, routing: MoeRouting, *, w2: Optional[torch.Tensor] = None,
    row_src: Optional[torch.Tensor] = None, row_scale: Optional[torch.Tensor] = None,
    row_scale_idx: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Grouped GEMM over ``routing``'s tile table. ``w`` is ``[E, N, K]`` (a view with contiguous K is
    fine). With ``w2`` the SwiGLU epilogue is fused and ``row_scale`` is required."""
    E, N, K = w.shape
    n_rows = routing.T * routing.k
    assert x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    assert x.stride(1) == 1 and w.stride(2) == 1
    if w2 is not None:
        assert w2.shape == w.shape and w2.stride() == w.stride() and row_scale is not None
    c = out if out is not None else _empty((n_rows, N), dtype=torch.bfloat16, device=x.device)
    _lib.check(
        _lib.load().vx_moe_gemm(
            x.data_ptr(), x.stride(0), w.data_ptr(), _ptr(w2), w.stride(1), w.stride(0), c.data_ptr(), c.stride(0),
            N, K, routing.tile_group.data_ptr(), routing.tile_row0.data_ptr(), routing.tile_rows.data_ptr(),
            routing.max_tiles, routing.bm, _ptr(row_src), _ptr(row_scale), _ptr(row_scale_idx),
            1 if w2 is not None else 0, x.shape[0], _stream(),
        ),
        "vx_moe_gemm",
    )
    return c


class PackedExpertWeights:
    """Fragment-order copy of ``[E, N, K]`` expert weights (``vx_pack_weights``) for the weight-streaming
    grouped GEMM at decode sizes. ``rows(a, b)`` names rows ``[a, b)`` of every expert (``a`` a multiple of 16)."""

    __slots__ = ("data", "E", "N", "K", "kchunks", "row0", "rows_n")

    def rows(self, a: int, b: int) -> "PackedExpertWeights":
        assert a % 16 == 0 and 0 <= a < b <= self.rows_n
        v = PackedExpertWeights()
        v.data, v.E, v.N, v.K, v.kchunks = self.data, self.E, self.N, self.K, self.kchunks
        v.row0, v.rows_n = self.row0 + a, b - a
        return v

    def data_ptr(self) -> int:
        return self.data.data_ptr() + (self.row0 // 16) * self.kchunks * 512 * 2

    @property
    def gstride(self) -> int:
        return ((self.N + 15) // 16) * self.kchunks * 512


def pack_expert_weights(w: torch.Tensor) -> PackedExpertWeights:
    """Pack ``w [E, N, K]`` (bf16, K contiguous, any row / expert pitch) into fragment order."""
    _need_gpu("w", w)
    assert w.dim() == 3 and w.dtype == torch.bfloat16 and w.stride(2) == 1
    E, N, K = w.shape
    lib = _lib.load()
    pk = PackedExpertWeights()
    pk.E, pk.N, pk.K, pk.kchunks, pk.row0, pk.rows_n = E, N, K, lib.vx_packed_kchunks(K), 0, N
    pk.data = _empty(E * pk.gstride, dtype=torch.bfloat16, device=w.device)
    _lib.check(lib.vx_pack_weights(w.data_ptr(), w.stride(1), w.stride(0), E, N, K, pk.data.data_ptr(), _stream()),
               "vx_pack_weights")
    return pk


def unpack_expert_weights(pk: PackedExpertWeights) -> torch.Tensor:
    """The ``[E, N, K]`` tensor that ``pk`` was packed from (for checkpointing or inspecting a model that holds
    fragment-order weights only; a permutation done with torch views, not a kernel)."""
    assert pk.row0 == 0 and pk.rows_n == pk.N, "unpack the whole tensor, not a row range"
    nb = (pk.N + 15) // 16
    v = pk.data.view(pk.E, nb, pk.kchunks, 4, 16, 8)  # [e][row block][k-chunk][lane / 16][lane % 16][8]
    return v.permute(0, 1, 4, 2, 3, 5).reshape(pk.E, nb * 16, pk.kchunks * 32)[:, : pk.N, : pk.K].contiguous()


def moe_gemm_packed(
    x: torch.Tensor, w: PackedExpertWeights, routing: MoeRouting, *, w2: Optional[PackedExpertWeights] = None,
    row_src: Optional[torch.Tensor] = None, row_scale: Optional[torch.Tensor] = None,
    row_scale_idx: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``moe_gemm`` on packed weights (tile tables of 16 / 32 / 64 rows: weight-streaming kernel; 256 rows:
    the 256 x 256 kernel, K a multiple of 64); same bits."""
    n_rows = routing.T * routing.k
    assert x.dtype == torch.bfloat16 and x.stride(1) == 1 and routing.bm in (16, 32, 64, 256)
    assert routing.bm != 256 or w.K % 64 == 0
    if w2 is not None:
        assert w2.data is w.data and w2.rows_n == w.rows_n and row_scale is not None
    N = w.rows_n
    c = out if out is not None else _empty((n_rows, N), dtype=torch.bfloat16, device=x.device)
    _lib.check(
        _lib.load().vx_moe_gemm_packed(
            x.data_ptr(), x.stride(0), w.data_ptr(), w2.data_ptr() if w2 is not None else None, w.gstride,
            c.data_ptr(), c.stride(0), N, w.K, routing.tile_group.data_ptr(), routing.tile_row0.data_ptr(),
            routing.tile_rows.data_ptr(), routing.max_tiles, routing.bm, _ptr(row_src), _ptr(row_scale),
            _ptr(row_scale_idx), 1 if w2 is not None else 0, x.shape[0], _stream(),
        ),
        "vx_moe_gemm_packed",
    )
    return c


def moe_gemm_nn(
    a: torch.Tensor, w: torch.Tensor, routing: MoeRouting, *, a_src: Optional[torch.Tensor] = None,
    a2: Optional[torch.Tensor] = None, w2: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Grouped data gradient: ``C[rows of e] = A[a_src[rows]] @ w[e] (+ A2[rows] @ w2[e])`` with ``w [E, K, N]``
    (N contiguous). ``routing`` has at most 128 rows per tile, or 256 (the wide kernel: K and w2's K multiples
    of 64); the bits do not depend on the tile height."""
    E, K, N = w.shape
    n_rows = routing.T * routing.k
    assert a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.stride(1) == 1 and w.stride(2) == 1
    assert a.shape[1] == K and (a_src is not None or a.shape[0] == n_rows)
    assert (a2 is None) == (w2 is None)
    K2 = 0
    if a2 is not None:
        K2 = w2.shape[1]
        assert a2.dtype == torch.bfloat16 and w2.dtype == torch.bfloat16 and a2.stride(1) == 1 and w2.stride(2) == 1
        assert a2.shape == (n_rows, K2) and w2.shape[0] == E and w2.shape[2] == N
    if a_src is not None:
        assert a_src.dtype == torch.int32 and a_src.is_contiguous() and a_src.numel() == n_rows
    c = out if out is not None else _empty((n_rows, N), dtype=torch.bfloat16, device=a.device)
    _lib.check(
        _lib.load().vx_moe_gemm_nn(
            a.data_ptr(), a.stride(0), _ptr(a_src), w.data_ptr(), w.stride(1), w.stride(0), K,
            _ptr(a2), a2.stride(0) if a2 is not None else 0, _ptr(w2), w2.stride(1) if w2 is not None else 0,
            w2.stride(0) if w2 is not None else 0, K2, c.data_ptr(), c.stride(0), N,
            routing.tile_group.data_ptr(), routing.tile_row0.data_ptr(), routing.tile_rows.data_ptr(),
            routing.max_tiles, routing.bm, a.shape[0], _stream(),
        ),
        "vx_moe_gemm_nn",
    )
    return c


def moe_gemm_tn(
    dy: torch.Tensor, x: torch.Tensor, cu: torch.Tensor, num_experts: int, *, dy_src: Optional[torch.Tensor] = None,
    x_src: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None, wide: bool = True,
) -> torch.Tensor:
    """Grouped weight gradient: ``dW[e] = dY[dy_src[r]]^T @ X[x_src[r]]`` summed over the sorted rows
    ``cu[e] <= r < cu[e + 1]``; returns ``[E, N, K]`` (zeros for an expert without rows). ``wide=False`` keeps
    the 128 x 128-tile kernel where the 256 x 256-tile one would run (same bits)."""
    N, K = dy.shape[1], x.shape[1]
    assert dy.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and dy.stride(1) == 1 and x.stride(1) == 1
    assert cu.dtype == torch.int32 and cu.is_contiguous() and cu.numel() == num_experts + 1
    for src in (dy_src, x_src):
        assert src is None or (src.dtype == torch.int32 and src.is_contiguous())
    dw = out if out is not None else _empty((num_experts, N, K), dtype=torch.bfloat16, device=dy.device)
    assert dw.shape == (num_experts, N, K) and dw.stride(2) == 1
    if dy.shape[0] == 0 or x.shape[0] == 0:  # no rows at all: every expert's gradient is zero
        return dw.zero_()
    _lib.check(
        _lib.load().vx_moe_gemm_tn(
            dy.data_ptr(), dy.stride(0), _ptr(dy_src), x.data_ptr(), x.stride(0), _ptr(x_src), dw.data_ptr(),
            dw.stride(1), dw.stride(0), N, K, cu.data_ptr(), num_experts, dy.shape[0] if wide else 0, x.shape[0] if wide else 0,
            _stream(),
        ),
        "vx_moe_gemm_tn",
    )
    return dw


def moe_swiglu_backward(g: torch.Tensor, u: torch.Tensor, d_hw: torch.Tensor, routing_weights: torch.Tensor,
                        sorted_flat: torch.Tensor, d_g_out: Optional[torch.Tensor] = None,
                        d_u_out: Optional[torch.Tensor] = None):
    """The elementwise step of the fused-MoE backward in one launch. ``g``, ``u``, ``d_hw`` are ``[T k, I]`` in
    sorted-row order (any row strides), ``routing_weights [T, k]`` bf16, ``sorted_flat`` the (token, slot) flat
    index of each sorted row. Returns ``(hw, d_g, d_u, d_routing_weights [T, k])``; ``d_g_out`` / ``d_u_out`` may
    be the two halves of one ``[T k, 2 I]`` buffer."""
    n, I = g.shape
    hw = _empty((n, I), dtype=torch.bfloat16, device=g.device)
    d_g = d_g_out if d_g_out is not None else _empty((n, I), dtype=torch.bfloat16, device=g.device)
    d_u = d_u_out if d_u_out is not None else _empty((n, I), dtype=torch.bfloat16, device=g.device)
    for t in (g, u, d_hw, d_g, d_u):
        assert t.dtype == torch.bfloat16 and t.shape == (n, I) and t.stride(1) == 1
    rw = routing_weights.contiguous()
    assert rw.dtype == torch.bfloat16 and rw.numel() == n and sorted_flat.dtype == torch.int32 and sorted_flat.numel() == n
    d_rw = _empty(rw.shape, dtype=torch.bfloat16, device=g.device)
    _lib.check(
        _lib.load().vx_moe_swiglu_bwd(
            g.data_ptr(), u.data_ptr(), d_hw.data_ptr(), g.stride(0), u.stride(0), d_hw.stride(0), rw.data_ptr(),
            sorted_flat.data_ptr(), hw.data_ptr(), d_g.data_ptr(), d_u.data_ptr(), d_rw.data_ptr(), hw.stride(0),
            d_g.stride(0), d_u.stride(0), n, I, _stream(),
        ),
        "vx_moe_swiglu_bwd",
    )
    return hw, d_g, d_u, d_rw


def expert_histogram(idx: torch.Tensor, num_bins: int) -> torch.Tensor:
    assert idx.is_cuda
    assert idx.dtype == torch.int32 or idx.dtype == torch.int64
    assert idx.numel() < (1 << 31) - 1, "Too many elements."
    flat = idx.flatten().contiguous()
    out = _empty(num_bins, dtype=torch.int32, device=idx.device)
    _lib.check(
        _lib.load().vx_expert_histogram(flat.data_ptr(), int(flat.dtype == torch.int64), flat.numel(), num_bins,
                                        out.data_ptr(), _stream()),
        "vx_expert_histogram",
    )
    return out


def moe_scatter(x: torch.Tensor, index: torch.Tensor, out_dtype=None) -> torch.Tensor:
    assert x.is_cuda and index.is_cuda
    assert x.shape[0] == index.shape[0]
    assert x.device == index.device, f"x.device = {x.device}, index.device = {index.device}"
    if x.dtype != torch.bfloat16 or (out_dtype or x.dtype) != torch.bfloat16:
        raise ValueError("moe_scatter supports bfloat16 only")
    M, N = x.shape
    topk = index.shape[1]
    idx = index.to(torch.int32).contiguous()
    xs = x if x.stride(1) == 1 else x.contiguous()
    out = _empty(M * topk, N, dtype=x.dtype, device=x.device)
    _lib.check(
        _lib.load().vx_moe_scatter(xs.data_ptr(), out.data_ptr(), idx.data_ptr(), M, topk, N, xs.stride(0),
                                   out.stride(0), _stream()),
        "vx_moe_scatter",
    )
    return out


def moe_gather(x: torch.Tensor, index: torch.Tensor, out_dtype=None, residual: Optional[torch.Tensor] = None,
               out: Optional[torch.Tensor] = None, norm_weight: Optional[torch.Tensor] = None,
               norm_out: Optional[torch.Tensor] = None, eps: float = 1e-6, hf_two_rounding: bool = True,
               prefetch: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``y[t] = sum_i x[index[t, i]]`` (fp32, slot order) ``(+ residual)``; with ``norm_weight`` and
    ``norm_out`` also writes ``norm_out = RMSNorm(y)`` in the same launch. ``prefetch``: a contiguous tensor
    (the next projection's weights) that spare workgroups read and discard meanwhile; changes no result."""
    assert x.is_cuda and index.is_cuda
    M, topk = index.shape
    assert x.shape[0] == M * topk
    assert x.device == index.device, f"x.device = {x.device}, index.device = {index.device}"
    if x.dtype != torch.bfloat16 or (out_dtype or x.dtype) != torch.bfloat16:
        raise ValueError("moe_gather supports bfloat16 only")
    N = x.shape[1]
    idx = index if (index.dtype == torch.int32 and index.is_contiguous()) else index.to(torch.int32).contiguous()
    xs = x if x.stride(1) == 1 else x.contiguous()
    y = out if out is not None else _empty(M, N, dtype=x.dtype, device=x.device)
    assert (norm_weight is None) == (norm_out is None)
    pf_bytes = 0
    if prefetch is not None:
        assert prefetch.is_contiguous() and prefetch.device == x.device
        pf_bytes = prefetch.numel() * prefetch.element_size()
    _lib.check(
        _lib.load().vx_moe_gather_norm_prefetch(
            xs.data_ptr(), idx.data_ptr(), _ptr(residual), y.data_ptr(), M, topk, N, xs.stride(0),
            residual.stride(0) if residual is not None else 0, y.stride(0), _ptr(norm_weight), _ptr(norm_out),
            norm_out.stride(0) if norm_out is not None else 0, float(eps), 1 if hf_two_rounding else 0,
            _ptr(prefetch), pf_bytes, _stream()),
        "vx_moe_gather_norm",
    )
    return y


def fused_moe(
    hidden_states: torch.Tensor,
    routing_weights: torch.Tensor,
    selected_experts: torch.Tensor,
    gate_w: torch.Tensor,
    up_w: torch.Tensor,
    down_w: torch.Tensor,
    num_experts: int,
    residual: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    packed: Optional[tuple] = None,
) -> torch.Tensor:
    """Router outputs -> expert SwiGLU MLPs -> slot-ordered combine, four launches:
    routing integers, gate/up grouped GEMM with gather-on-load and fused SiLU*up*weight,
    down grouped GEMM, fp32 slot-order sum. ``packed`` = (``pack_expert_weights`` of the stacked
    ``[E, 2I, H]`` gate/up weight, of ``down_w``): read instead of the tensors when the step's expert
    tiles have at most 64 rows (same bits)."""
    T, H = hidden_states.shape
    k = selected_experts.shape[1]
    x = hidden_states if hidden_states.stride(1) == 1 else hidden_states.contiguous()
    rw = routing_weights.contiguous()
    H_, I_ = gate_w.shape[-1], down_w.shape[-1]
    r = moe_route(selected_experts, num_experts,
                  bm=moe_tile_rows(selected_experts.shape[0], wide_ok=(H_ % 64 == 0 and I_ % 64 == 0),
                                   packed=packed is not None, top_k=k, num_experts=num_experts))
    if packed is not None and (r.bm <= 64 or r.bm == 256):
        pgu, pdn = packed
        assert pgu.rows_n == 2 * I_ and pgu.K == H_ and pdn.rows_n == down_w.shape[1] and pdn.K == I_
        hw = moe_gemm_packed(x, pgu.rows(0, I_), r, w2=pgu.rows(I_, 2 * I_), row_src=r.sorted_token, row_scale=rw,
                             row_scale_idx=r.sorted_flat)
        o = moe_gemm_packed(hw, pdn, r)
    else:
        hw = moe_gemm(x, gate_w, r, w2=up_w, row_src=r.sorted_token, row_scale=rw, row_scale_idx=r.sorted_flat)
        o = moe_gemm(hw, down_w, r)
    return moe_gather(o, r.scatter_index, residual=residual, out=out)


# ----------------------------------------------------------------------------- decoder glue


def qk_norm_rope_store(qkv, q_norm_w, k_norm_w, cos_table, sin_table, positions, slot_mapping, q_out,
                       k_cache, v_cache, Hq: int, Hkv: int, D: int, eps: float, k_out=None) -> None:
    """Caches are ``[blocks, page, Hkv, D]`` views (any block / row / head strides, D contiguous).
    ``positions=None``: ``cos_table`` / ``sin_table`` hold one row per token."""
    T = qkv.shape[0]
    assert qkv.stride(1) == 1 and qkv.shape[1] == (Hq + 2 * Hkv) * D
    assert cos_table.is_contiguous() and sin_table.is_contiguous() and cos_table.shape == sin_table.shape
    assert cos_table.shape[1] == D and cos_table.dtype == torch.bfloat16 and sin_table.dtype == torch.bfloat16
    if positions is None:
        assert cos_table.shape[0] >= T
    else:
        assert positions.dtype in (torch.int32, torch.int64)
    page, sb, sp, sh = 1, 0, 0, 0
    if k_cache is not None:
        assert k_cache.dim() == 4 and k_cache.shape[2] == Hkv and k_cache.shape[3] == D and k_cache.stride(3) == 1
        page, (sb, sp, sh) = k_cache.shape[1], k_cache.stride()[:3]
        if v_cache is not None:
            assert v_cache.shape == k_cache.shape and v_cache.stride() == k_cache.stride()
    _lib.check(
        _lib.load().vx_qk_norm_rope_store(
            qkv.data_ptr(), qkv.stride(0), q_norm_w.data_ptr(), k_norm_w.data_ptr(), cos_table.data_ptr(),
            sin_table.data_ptr(), _ptr(positions), int(positions is not None and positions.dtype == torch.int64),
            _ptr(slot_mapping),
            q_out.data_ptr(), _ptr(k_out), _ptr(k_cache), _ptr(v_cache), T, Hq, Hkv, D, float(eps),
            cos_table.shape[0], page, sb, sp, sh, _stream(),
        ),
        "vx_qk_norm_rope_store",
    )


def rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotary embedding of ``x [T, H, D]`` (bf16, D contiguous, any token / head strides) with per-token rows
    ``cos`` / ``sin [T, D]``: HuggingFace's ``x * cos + rotate_half(x) * sin`` with its bf16 roundings, one
    launch. Returns a contiguous ``[T, H, D]`` tensor."""
    _need_gpu("x", x)
    assert x.dim() == 3 and x.dtype == torch.bfloat16 and x.stride(2) == 1
    T, H, D = x.shape
    assert cos.shape == (T, D) and sin.shape == (T, D) and cos.dtype == torch.bfloat16 and sin.dtype == torch.bfloat16
    if cos.stride(1) != 1 or sin.stride() != cos.stride():
        cos, sin = cos.contiguous(), sin.contiguous()
    out = _empty((T, H, D), dtype=x.dtype, device=x.device)
    _lib.check(
        _lib.load().vx_rope(x.data_ptr(), out.data_ptr(), cos.data_ptr(), sin.data_ptr(), T, H, D, x.stride(0), x.stride(1),
                            out.stride(0), out.stride(1), cos.stride(0), _stream()),
        "vx_rope",
    )
    return out


def embedding(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    T = ids.numel()
    vocab, H = table.shape
    o = out if out is not None else _empty((T, H), dtype=table.dtype, device=table.device)
    _lib.check(
        _lib.load().vx_embedding(table.data_ptr(), ids.data_ptr(), int(ids.dtype == torch.int64), o.data_ptr(), T, H,
                                 vocab, _stream()),
        "vx_embedding",
    )
    return o
