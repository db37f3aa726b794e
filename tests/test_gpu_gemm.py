"""GPU parity: batch-invariant GEMM. Restates tests/batch_invariant_ops/test_matmul.py:25-46 (row
slice vs full batch, atol = rtol = 0) and the linspace variant of
tests/batch_invariant_ops/test_batch_invariance.py:30-44, plus parity with the CPU oracle."""

import pytest
import torch

from oracle import row_ops as O
from tests.util import assert_bf16_close, assert_bitwise, bf16_ulp_distance

pytestmark = pytest.mark.gpu

from vexact_amd import ops  # noqa: E402
from vexact_amd.batch_invariant_ops import matmul_persistent, set_batch_invariant_mode, triton_bmm  # noqa: E402


def _gen(shape, seed, dtype=torch.bfloat16, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("K,N", [(2048, 4096), (4096, 2048), (2048, 128), (768, 2048), (136, 200)])
def test_bf16_linear_bits_do_not_depend_on_batch(K, N):
    a = _gen((300, K), 1)
    w = _gen((N, K), 2, scale=0.02)
    ag, wg = a.cuda(), w.cuda()
    full = matmul_persistent(ag, wg.t())
    assert_bf16_close(full, O.matmul_ref(a, w.t()), max_ulp=2, what=f"mm {K}x{N} vs oracle")
    for m in (1, 7, 16, 17, 33, 64, 65, 128, 256):
        assert_bitwise(matmul_persistent(ag[:m], wg.t()), full[:m], f"mm first {m} rows")
    assert_bitwise(matmul_persistent(ag[200:201], wg.t()), full[200:201], "mm row 200 alone")
    assert_bitwise(matmul_persistent(ag[129:140], wg.t()), full[129:140], "mm rows 129..139")


def test_stream_and_tiled_kernels_agree_bitwise():
    a = _gen((130, 1024), 3)
    w = _gen((328, 1024), 4, scale=0.05)
    bias = _gen((328,), 5)
    ag, wg, bg = a.cuda(), w.cuda(), bias.cuda()
    ref = ops.gemm_nt_variant(ag, wg, kind=1, bias=bg)
    for mt in (1, 2, 4):
        assert_bitwise(ops.gemm_nt_variant(ag, wg, kind=0, mt=mt, bias=bg), ref, f"stream mt={mt} vs tiled")
    assert_bf16_close(ref, O.matmul_ref(a, w.t(), bias), max_ulp=2, what="biased gemm vs oracle")


@pytest.mark.parametrize("K", [8, 16, 24, 40])
@pytest.mark.parametrize("M", [1, 17, 64])
def test_streaming_and_tiled_kernels_on_contraction_depths_below_their_step(M, K):
    # K below the streaming kernel's 32-wide step (and the tiled kernel's 64): the pieces of a step that lie past K
    # are replaced by a re-read of the row's first piece and zeroed, so nothing outside the row is touched. The weight
    # tensor ends where its allocation ends, the case in which a read past the last row would leave mapped memory.
    N = 80
    a = _gen((M, K), 40 + K)
    w = _gen((N, K), 41 + K, scale=0.3)
    ag, wg = a.cuda(), w.cuda()
    ref = ops.gemm_nt_variant(ag, wg, kind=1)
    for mt in (1, 2, 4):
        assert_bitwise(ops.gemm_nt_variant(ag, wg, kind=0, mt=mt), ref, f"stream mt={mt} vs tiled at K={K}")
    assert_bf16_close(ref, O.matmul_ref(a, w.t()), max_ulp=2, what=f"K={K} vs oracle")


@pytest.mark.parametrize(
    "M,N,K,bias",
    [
        (256, 256, 64, False),  # one tile, one k-step
        (300, 520, 128, True),  # ragged rows and columns, two k-steps
        (513, 1023, 192, False),  # row stride of C not a multiple of 8 -> scalar stores
        (4352, 4096, 128, False),  # 272 tiles on 256 workgroups: some walk a second tile
        (2048, 5120, 2048, True),  # qkv-projection shape of a prefill chunk
        (2000, 10240, 128, True),  # 8 x 40 tiles: columns from 8192 on go to 128-row tiles (ragged last row tile)
        (256, 152000, 64, False),  # 594 column tiles: the last 82 go to 128-row tiles (ragged last column tile)
        (8192, 5120, 64, True),  # 32 x 20 tiles: two rounds of 256-row tiles and one of 128-row tiles
    ],
)
def test_wide_kernel_agrees_bitwise(M, N, K, bias):
    a = _gen((M, K), 13)
    w = _gen((N, K), 14, scale=0.05)
    ag, wg = a.cuda(), w.cuda()
    bg = _gen((N,), 15).cuda() if bias else None
    ref = ops.gemm_nt_variant(ag, wg, kind=1, bias=bg)
    assert_bitwise(ops.gemm_nt_variant(ag, wg, kind=3, bias=bg), ref, f"wide vs tiled {M}x{N}x{K}")
    if M * N >= 128 * 65536:  # the default entry point picks the wide kernel here
        full = ops.gemm_nt(ag, wg, bias=bg)
        assert_bitwise(full, ref, "dispatch vs tiled")
        r0 = min(1000, M // 2)
        assert_bitwise(ops.gemm_nt(ag[r0 : r0 + 3], wg, bias=bg), full[r0 : r0 + 3], "3 rows alone vs inside a chunk")


def test_dispatch_agrees_with_the_tiled_kernel_on_random_shapes():
    # whatever kernel the shape-based dispatch picks (streaming, ring at 1..512 rows, 128 x 128 tiles, 256 x 256
    # tiles with or without a half-height last round), the bits are those of the 128 x 128 tiled kernel, with
    # strided operands and a bias as well
    g = torch.Generator().manual_seed(77)
    def pick(choices):
        return choices[int(torch.randint(0, len(choices), (1,), generator=g))]
    shapes = [(1, 2048, 4096), (16, 128, 2048), (48, 5120, 2048), (64, 8192, 256), (64, 8256, 256), (33, 1000, 192),
              (65, 136, 72), (300, 5120, 64), (2304, 7168, 64), (1100, 10240, 128)]
    for _ in range(14):
        shapes.append((int(torch.randint(1, 700, (1,), generator=g)), 8 * int(torch.randint(1, 1200, (1,), generator=g)),
                       pick([64, 72, 128, 192, 256, 320, 1024, 2048])))
    for i, (M, N, K) in enumerate(shapes):
        pad_x, pad_w = pick([0, 8, 64]), pick([0, 8, 64])
        a = _gen((M, K + pad_x), 100 + i)[:, :K].cuda()
        w = _gen((N, K + pad_w), 200 + i, scale=0.05)[:, :K].cuda()
        bias = _gen((N,), 300 + i).cuda() if i % 2 else None
        ref = ops.gemm_nt_variant(a.contiguous(), w.contiguous(), kind=1, bias=bias)
        assert_bitwise(ops.gemm_nt(a, w, bias=bias), ref, f"dispatch vs tiled, {M}x{N}x{K}, row pads {pad_x}/{pad_w}")


@pytest.mark.parametrize("M,N,K", [(256, 640, 2048), (100, 200, 64), (77, 333, 192), (130, 70, 320), (512, 128, 768),
                                   (3000, 128, 512)])  # the last: many rows, few columns -> ring by dispatch
def test_ring_kernel_agrees_bitwise(M, N, K):
    a = _gen((M, K), 16)
    w = _gen((N, K), 17, scale=0.05)
    bias = _gen((N,), 18)
    ag, wg, bg = a.cuda(), w.cuda(), bias.cuda()
    ref = ops.gemm_nt_variant(ag, wg, kind=1, bias=bg)
    ran = 0
    for cfg, kdiv in ((0, 64), (1, 128), (2, 128), (3, 128), (4, 256), (5, 64), (6, 64)):
        if K % kdiv:
            continue
        assert_bitwise(ops.gemm_nt_variant(ag, wg, kind=4, mt=cfg, bias=bg), ref, f"ring config {cfg} vs tiled")
        ran += 1
    assert ran >= 3
    assert_bitwise(ops.gemm_nt(ag, wg, bias=bg), ref, "dispatch vs tiled")


def test_lm_head_shape_rows():
    # config-1 shaped: [M, 2048] x [2048, 151936], rows of one draw
    a = _gen((64, 2048), 6)
    w = _gen((151936, 2048), 7, scale=0.02)
    ag, wg = a.cuda(), w.cuda()
    full = matmul_persistent(ag, wg.t())
    for m in (1, 7):
        assert_bitwise(matmul_persistent(ag[:m], wg.t()), full[:m], f"lm_head first {m}")
    ref = O.matmul_ref(a[:4], w.t())
    assert_bf16_close(full[:4], ref, max_ulp=2, what="lm_head vs oracle")


def test_linspace_inputs():
    a = torch.linspace(-100, 100, 32 * 512).reshape(32, 512).to(torch.bfloat16).cuda()
    b = torch.linspace(-100, 100, 512 * 64).reshape(512, 64).to(torch.bfloat16).cuda()
    full = matmul_persistent(a, b)
    assert_bitwise(matmul_persistent(a[:1], b), full[:1], "linspace row 0")
    assert_bf16_close(full, O.matmul_ref(a.cpu(), b.cpu()), max_ulp=2, what="linspace vs oracle")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.float16, 2e-3)])
def test_other_dtypes_and_layouts(dtype, tol):
    a = _gen((37, 100), 8, dtype)
    b = _gen((100, 53), 9, dtype)
    bias = _gen((53,), 10, dtype)
    got = matmul_persistent(a.cuda(), b.cuda(), bias.cuda())
    ref = O.matmul_ref(a, b, bias)
    torch.testing.assert_close(got.cpu().float(), ref.float(), atol=tol * 10, rtol=tol)
    assert_bitwise(matmul_persistent(a[:1].cuda(), b.cuda(), bias.cuda()), got[:1], "generic row 0")
    # bf16, K not a multiple of 8 -> generic kernel; transposed a
    a2 = _gen((100, 37), 11).t()
    b2 = _gen((100, 53), 12)
    got2 = matmul_persistent(a2.cuda(), b2.cuda())
    assert_bf16_close(got2, O.matmul_ref(a2, b2), max_ulp=2, what="generic bf16")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("M,N,K,bias,linear_layout", [
    (300, 520, 256, True, True),     # nn.Linear layout, vector loads
    (65, 100, 100, False, False),    # row-major b (made K-contiguous), ragged everything
    (130, 77, 1031, True, True),     # K not a multiple of the vector width: scalar loads
    (1, 2048, 2048, False, True),
])
def test_fp32_fp16_matrix_core_gemm(dtype, M, N, K, bias, linear_layout):
    # the fp16 / fp32 configurations of matmul_persistent (batch_invariant_ops.py:182-206): rows do not depend on the
    # batch (0 bits), results against an fp64 product of the same inputs
    a = _gen((M, K), 21, dtype)
    w = _gen((N, K), 22, dtype, scale=0.1)
    bv = _gen((N,), 23, dtype) if bias else None
    ag, wg = a.cuda(), w.cuda()
    bmat = wg.t() if linear_layout else wg.t().contiguous()
    full = matmul_persistent(ag, bmat, bv.cuda() if bias else None)
    assert full.dtype == dtype and full.shape == (M, N)
    want = a.double() @ w.double().t() + (bv.double() if bias else 0.0)
    err = (full.cpu().double() - want).abs().max().item()
    scale = want.abs().max().item()
    if dtype == torch.float32:
        assert err <= 2e-6 * scale * (K ** 0.5), (err, scale)   # true fp32 products and sums
        tf32_err = ((a.double() @ w.double().t()) * 2.0 ** -11).abs().max().item()
        assert err < 0.1 * tf32_err, "fp32 GEMM must not run at TF32 precision"
    else:
        got, ref16 = full.cpu(), want.to(torch.float16)
        ulp = (got.view(torch.int16).int() - ref16.view(torch.int16).int()).abs()
        same_sign = (got.view(torch.int16).int() ^ ref16.view(torch.int16).int()) >= 0
        assert bool(((ulp <= 2) & same_sign | ((got.double() - want).abs() <= 2e-3 * scale)).all()), "fp16 beyond 2 ulp"
    for m in sorted({1, 7, 33, 64, 65, M} & set(range(1, M + 1))):
        assert_bitwise(matmul_persistent(ag[:m], bmat, bv.cuda() if bias else None), full[:m], f"{dtype} first {m} rows")
    if M > 40:
        assert_bitwise(matmul_persistent(ag[37:40], bmat, bv.cuda() if bias else None), full[37:40], f"{dtype} rows 37..39 alone")
    # under the aten overrides
    with set_batch_invariant_mode(True):
        via_aten = torch.mm(ag, bmat) if not bias else torch.addmm(bv.cuda(), ag, bmat)
    assert_bitwise(via_aten, full, f"{dtype} through aten::mm / addmm")


def test_aten_overrides_and_mode_switch():
    from vexact_amd.batch_invariant_ops import (
        disable_batch_invariant_mode,
        enable_batch_invariant_mode,
        is_batch_invariant_mode_enabled,
    )

    a = _gen((64, 256), 13).cuda()
    lin = torch.nn.Linear(256, 512, bias=True, dtype=torch.bfloat16, device="cuda")
    assert not is_batch_invariant_mode_enabled()
    with set_batch_invariant_mode(True):
        assert is_batch_invariant_mode_enabled()
        y = lin(a)
        y1 = lin(a[:1])
        assert_bitwise(y1, y[:1], "nn.Linear under the override")
        assert_bitwise(y, matmul_persistent(a, lin.weight.t(), lin.bias), "override == direct call")
        m = torch.mm(a, lin.weight.t())
        assert_bitwise(m, matmul_persistent(a, lin.weight.t()), "aten::mm override")
        x32 = a.float().pow(2)
        assert_bitwise(x32.mean(-1, keepdim=True), ops.mean_dim(x32, -1, keepdim=True), "aten::mean.dim override")
        ls = torch.log_softmax(a.float(), dim=-1)
        assert_bitwise(ls, ops.log_softmax(a.float()), "aten::_log_softmax override")
        with set_batch_invariant_mode(False):
            assert not is_batch_invariant_mode_enabled()
        assert is_batch_invariant_mode_enabled()
        assert_bitwise(torch.mm(a, lin.weight.t()), m, "override restored after nested disable")
    assert not is_batch_invariant_mode_enabled()
    enable_batch_invariant_mode()
    enable_batch_invariant_mode()
    assert is_batch_invariant_mode_enabled()
    disable_batch_invariant_mode()
    assert not is_batch_invariant_mode_enabled()
    enable_batch_invariant_mode()
    assert_bitwise(torch.mm(a, lin.weight.t()), m, "enable -> disable -> enable")
    disable_batch_invariant_mode()
    torch.use_deterministic_algorithms(False)


def test_bmm():
    a = _gen((3, 5, 16), 14, torch.float32)
    b = _gen((3, 16, 9), 15, torch.float32)
    got = triton_bmm(a.cuda(), b.cuda())
    torch.testing.assert_close(got.cpu(), torch.bmm(a, b), atol=1e-5, rtol=1e-5)
    inv = _gen((1, 32, 1), 16, torch.float32)
    pos = torch.arange(40, dtype=torch.float32).reshape(1, 1, 40)
    got = triton_bmm(inv.cuda(), pos.cuda())
    torch.testing.assert_close(got.cpu(), torch.bmm(inv, pos), atol=0, rtol=0)  # single products are exact
    with pytest.raises(AssertionError):
        triton_bmm(a.cuda()[0], b.cuda())


@pytest.mark.parametrize("N,K", [(1536, 2048), (6144, 1024), (200, 264)])
def test_dense_swiglu_equals_unfused_chain_and_is_row_invariant(N, K):
    g = torch.Generator(device="cuda").manual_seed(N + K)
    wg = torch.empty(N, K, dtype=torch.bfloat16, device="cuda").normal_(0, 0.03, generator=g)
    wu = torch.empty(N, K, dtype=torch.bfloat16, device="cuda").normal_(0, 0.03, generator=g)
    xall = torch.empty(4096, K, dtype=torch.bfloat16, device="cuda").normal_(0, 1.0, generator=g)
    big = ops.gemm_swiglu(xall, wg, wu)                       # 4096 rows: wide or tiled kernel
    for M in (1, 7, 64, 65, 300, 384, 385, 2048):
        print(f"[case] dense swiglu M={M} N={N} K={K}", flush=True)
        x = xall[:M]
        got = ops.gemm_swiglu(x, wg, wu)
        assert_bitwise(got, big[:M], f"rows 0..{M} alone vs inside 4096 rows")
        gate, up = ops.gemm_nt(x, wg), ops.gemm_nt(x, wu)
        want = torch.nn.functional.silu(gate) * up            # bf16 silu, bf16 multiply
        ulp = bf16_ulp_distance(got, want)
        assert int(ulp.max()) <= 1 and float((ulp == 0).float().mean()) > 0.999, (int(ulp.max()), float((ulp == 0).float().mean()))
    # every kernel that can run the shape gives the same bits
    x = xall[:300]
    ref = ops.gemm_swiglu(x, wg, wu)
    for kind, mt in ((0, 1), (0, 2), (0, 4), (1, 0)) + (((3, 0),) if K % 64 == 0 else ()):
        assert_bitwise(ops.gemm_swiglu(x, wg, wu, kind=kind, mt=mt), ref, f"kind {kind} mt {mt}")
    # and the fused MoE's expert MLP with routing weight 1 is the same arithmetic
    down = torch.empty(256, N, dtype=torch.bfloat16, device="cuda").normal_(0, 0.03, generator=g)
    y = ops.swiglu_mlp(x, wg, wu, down)
    assert_bitwise(y, ops.gemm_nt(ref, down), "swiglu_mlp")


@pytest.mark.parametrize("M,N,K", [(4096, 2048, 1000), (2048, 4096, 8192), (2560, 2560, 64), (4096, 2048, 8)])
def test_weight_gradient_layout_gives_the_bits_of_the_transposed_copies(M, N, K):
    # matmul(d_y.t(), x): both operands with the contraction index slow go to the grouped weight-gradient kernel as
    # they lie; the same product through transposed copies and the NT kernels must give the same bits
    g = torch.Generator().manual_seed(M + K)
    dy = torch.randn(K, M, generator=g).to(torch.bfloat16).cuda()
    x = torch.randn(K, N, generator=g).to(torch.bfloat16).cuda()
    direct = ops.matmul(dy.t(), x)
    copies = ops.gemm_nt(dy.t().contiguous(), x.t().contiguous())
    assert_bitwise(direct, copies, "d_y^T x: grouped kernel vs transposed copies")


@pytest.mark.parametrize("M,N,K", [(4096, 2048, 4096), (1024, 520, 64), (1500, 2048, 512)])
def test_data_gradient_layout_gives_the_bits_of_the_transposed_copy(M, N, K):
    # matmul(d_y, w) with w row-major [K, N]: the grouped data-gradient kernel with one group, against the NT kernels
    # on a transposed copy of w; rows alone give the same bits (the choice of kernel by M changes nothing)
    g = torch.Generator().manual_seed(M + N)
    dy = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(K, N, generator=g) * 0.05).to(torch.bfloat16).cuda()
    direct = ops.matmul(dy, w)
    assert_bitwise(direct, ops.gemm_nt(dy, w.t().contiguous()), "d_y w: grouped kernel vs transposed copy")
    assert_bitwise(ops.matmul(dy[300:337].contiguous(), w), direct[300:337], "rows 300..336 alone")
