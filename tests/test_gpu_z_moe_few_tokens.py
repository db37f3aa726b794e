"""GPU parity: the expert GEMMs of a step of a few tokens (16-row tiles, one-wavefront blocks) against 32-row tiles.

Collected after the other kernel tests: the dispatch rule it exercises (one-wavefront blocks for 16-row tiles when the
4-wavefront blocks would be few and the contraction depth is at least 1024) was last changed after the final GPU run of the
full suite.
"""

import pytest
import torch

from oracle import moe as OM
from tests.util import assert_bitwise

pytestmark = pytest.mark.gpu

from vexact_amd import ops  # noqa: E402


def _inputs(T, H, I, E, k, seed, w_scale=0.02):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w, sel = OM.router_ref(torch.randn(T, E, generator=g), k)
    gate = (torch.randn(E, I, H, generator=g) * w_scale).to(torch.bfloat16)
    up = (torch.randn(E, I, H, generator=g) * w_scale).to(torch.bfloat16)
    down = (torch.randn(E, H, I, generator=g) * w_scale).to(torch.bfloat16)
    return x, w, sel, gate, up, down


@pytest.mark.parametrize("T,H,I,E,k", [(1, 2048, 768, 128, 8), (4, 2048, 768, 128, 8), (3, 1024, 200, 16, 4), (2, 1104, 72, 8, 2),
                                       (2, 256, 1024, 8, 2), (5, 1024, 1032, 6, 3)])
def test_one_wavefront_blocks_for_a_few_tiles_give_the_same_bits(T, H, I, E, k):
    # A step of a few tokens on 16-row tiles with a contraction depth of at least 1024 is launched as one-wavefront
    # blocks of 16 weight rows (gate/up at H >= 1024, down at I >= 1024; ragged N = 200 / 72, K = 1104 / 1032 included).
    # 32-row tiles never are, so they are the yardstick; tensors and fragment-order copies alike.
    assert ops.moe_tile_rows(T, top_k=k, num_experts=E) == 16
    x, w, sel, gate, up, down = _inputs(T, H, I, E, k, seed=43)
    xg, wg, sg, dg = x.cuda(), w.cuda(), sel.cuda(), down.cuda()
    gu = torch.cat([gate, up], dim=1).cuda()
    packable = I % 16 == 0
    if packable:
        pgu, pdn = ops.pack_expert_weights(gu), ops.pack_expert_weights(dg)
    res = {}
    for bm in (16, 32):
        r = ops.moe_route(sg, E, bm=bm)
        hw = ops.moe_gemm(xg, gu[:, :I, :], r, w2=gu[:, I:, :], row_src=r.sorted_token, row_scale=wg, row_scale_idx=r.sorted_flat)
        eo = ops.moe_gemm(hw, dg, r)
        res[bm] = (hw, eo)
        if packable:
            hw_p = ops.moe_gemm_packed(xg, pgu.rows(0, I), r, w2=pgu.rows(I, 2 * I), row_src=r.sorted_token, row_scale=wg,
                                       row_scale_idx=r.sorted_flat)
            eo_p = ops.moe_gemm_packed(hw, pdn, r)
            assert_bitwise(hw_p, hw, f"gate/up on packed weights, {bm}-row tiles")
            assert_bitwise(eo_p, eo, f"down on packed weights, {bm}-row tiles")
    assert_bitwise(res[16][0], res[32][0], "gate/up + SwiGLU, 16-row tiles in one-wavefront blocks against 32-row tiles")
    assert_bitwise(res[16][1], res[32][1], "down projection, 16-row tiles in one-wavefront blocks against 32-row tiles")
    # the whole block (which picks 16-row tiles by itself at these token counts) against the same block on 32-row tiles
    out = ops.fused_moe(xg, wg, sg, gu[:, :I, :], gu[:, I:, :], dg, E)
    r32 = ops.moe_route(sg, E, bm=32)
    assert_bitwise(out, ops.moe_gather(res[32][1], r32.scatter_index), "fused MoE block on a few tokens")
