"""Host-side logic that needs no GPU: step metadata, bucket padding, block allocator, contexts."""

import threading
import types

import numpy as np
import pytest
import torch

from oracle import metadata as OMeta
from vexact_amd.batch_invariant_ops import AttentionBlockSize, get_batch_invariant_attention_block_size
from vexact_amd.batch_invariant_ops import kv_cache_context as KC
from vexact_amd.decoder import StepBuffers, build_step_metadata, capture_sizes, decode_bytes_per_step, qwen3_30b_a3b, tiny_config


def _requests(rng, n, page):
    reqs, nxt = [], 0
    for _ in range(n):
        done = int(rng.integers(1, 200))
        this = int(rng.integers(1, done + 1)) if rng.random() < 0.5 else 1
        nb = (done + page - 1) // page
        ids = list(range(nxt, nxt + nb))
        rng.shuffle(ids)
        nxt += nb
        reqs.append(dict(num_computed_tokens=done, tokens_this_step=this, block_ids=ids))
    return reqs


def test_step_metadata_matches_the_loop_restatement():
    rng = np.random.default_rng(0)
    for page in (16, 256, 5):
        reqs = _requests(rng, 9, page)
        got = build_step_metadata(reqs, page, 40)
        ref = OMeta.prepare_gen_ctx_ref(reqs, page, 40)
        for k in ("slot_mapping", "context_lens", "block_tables", "query_start_loc", "positions"):
            assert np.array_equal(got[k], ref[k]), k
            assert got[k].dtype == ref[k].dtype, k
        assert got["max_seqlen_q"] == ref["max_seqlen_q"]


def test_hand_worked_metadata_example():
    # page 4; request A has 6 tokens cached in blocks [7, 2] and adds 1; request B prefills 3 into block [5]
    reqs = [dict(num_computed_tokens=7, tokens_this_step=1, block_ids=[7, 2]),
            dict(num_computed_tokens=3, tokens_this_step=3, block_ids=[5])]
    m = OMeta.prepare_gen_ctx_ref(reqs, 4, 3)
    assert m["slot_mapping"].tolist() == [2 * 4 + 2, 20, 21, 22]
    assert m["positions"].tolist() == [6, 0, 1, 2]
    assert m["context_lens"].tolist() == [7, 3]
    assert m["block_tables"].tolist() == [[7, 2, -1], [5, -1, -1]]
    assert m["query_start_loc"].tolist() == [0, 1, 4] and m["max_seqlen_q"] == 3


def test_hand_worked_graph_padding_example():
    # Literal pin of the padding restatement (vexact/inferencer/inferencer.py:306-324), worked by hand from the
    # reference's statements: buffers zeroed / filled with -1, the step copied in, then rows of padded requests zeroed
    # in the block table and their query_start_loc set to the real token count. Page 4, three requests, a bucket of
    # 8 tokens and 5 sequences, table rows of 4 blocks.
    reqs = [dict(num_computed_tokens=6, tokens_this_step=2, block_ids=[5, 2]),       # positions 4, 5 -> block 2 rows 0, 1
            dict(num_computed_tokens=1, tokens_this_step=1, block_ids=[7]),          # position 0 -> block 7 row 0
            dict(num_computed_tokens=9, tokens_this_step=3, block_ids=[0, 3, 9])]    # positions 6, 7, 8 -> block 3 rows 2, 3; block 9 row 0
    want = dict(slot_mapping=[8, 9, 28, 14, 15, 36, -1, -1],       # slot_mapping.fill_(-1), [:6] copied
                positions=[4, 5, 0, 6, 7, 8, 0, 0],                # position_ids zeroed, [:6] copied
                context_lens=[6, 1, 9, 0, 0],                      # context_lens zeroed, [:3] copied
                block_tables=[[5, 2, -1, -1], [7, -1, -1, -1], [0, 3, 9, -1], [0, 0, 0, 0], [0, 0, 0, 0]],
                query_start_loc=[0, 2, 3, 6, 6, 6])                # [num_seqs + 1 : graph_num_seqs + 1] = total_tokens
    ref = OMeta.pad_for_graph_ref(OMeta.prepare_gen_ctx_ref(reqs, 4, 4), 8, 5)
    for k, v in want.items():
        assert ref[k].tolist() == v, k
    assert ref["max_seqlen_q"] == 3
    # the product against the same literals: the Python builder + StepBuffers.load, and the one-pass native builder
    cfg = tiny_config()
    cfg.page_size, cfg.max_model_len = 4, 16
    b = StepBuffers(cfg, 8, 5, "cpu")
    assert b.load(build_step_metadata(reqs, 4, 4), np.arange(6))[:2] == (6, 3)
    for k, v in want.items():
        assert getattr(b, k).tolist() == v, k
    b2 = StepBuffers(cfg, 8, 5, "cpu")
    b2.meta_host.fill_(0x5A)
    assert b2.load_requests(reqs, np.arange(6), 4) == (6, 3, 3)
    for k, v in want.items():
        assert getattr(b2, k).tolist() == v, k


def test_hand_worked_block_allocator_restatement():
    # The scan restatement itself (vexact/batch_invariant_ops/kv_cache_context.py:177-217) on a hand-worked sequence:
    # min() of the free set per block, nothing allocated when the request does not fit, frees of ids that are not
    # allocated ignored, freed ids handed out again lowest first.
    r = OMeta.BlockAllocatorRef(6, 4)
    assert r.allocate(9) == [0, 1, 2]                   # ceil(9 / 4) = 3 blocks
    assert r.allocate(9, 3) == []                       # already covered
    assert r.allocate(13, 3) == [3]                     # one more block
    assert r.allocate(100) is None and sorted(r.free) == [4, 5] and sorted(r.allocated) == [0, 1, 2, 3]
    r.release([1, 3, 3, 5])                             # 3 twice: second ignored; 5 was never allocated: ignored
    assert sorted(r.free) == [1, 3, 4, 5] and sorted(r.allocated) == [0, 2]
    assert r.allocate(8) == [1, 3]
    assert r.allocate(4) == [4]
    assert r.allocate(0) == [] and r.allocate(5, 2) == []
    assert r.allocate(8) is None and sorted(r.free) == [5]   # two needed, one free: None and nothing taken


def test_bucket_padding_rules():
    cfg = tiny_config()
    rng = np.random.default_rng(1)
    reqs = _requests(rng, 3, cfg.page_size)
    for r in reqs:
        r["tokens_this_step"] = 1
    meta = build_step_metadata(reqs, cfg.page_size, cfg.max_model_len // cfg.page_size)
    b = StepBuffers(cfg, 8, 8, "cpu")
    T, B = b.load(meta, np.array([11, 12, 13]))
    ref = OMeta.pad_for_graph_ref(meta, 8, 8)
    assert (T, B) == (3, 3)
    assert b.input_ids.tolist() == [11, 12, 13, 0, 0, 0, 0, 0]
    assert np.array_equal(b.slot_mapping.numpy(), ref["slot_mapping"])
    assert np.array_equal(b.positions.numpy(), ref["positions"])
    assert np.array_equal(b.context_lens.numpy(), ref["context_lens"])
    assert np.array_equal(b.block_tables.numpy(), ref["block_tables"])
    assert np.array_equal(b.query_start_loc.numpy(), ref["query_start_loc"])
    assert b.seq_order.tolist() == sorted(range(8), key=lambda s: (-int(ref["context_lens"][s]), s))
    with pytest.raises(ValueError, match="total_tokens exceeds capture_tokens"):
        StepBuffers(cfg, 2, 8, "cpu").load(meta, np.array([1, 2, 3]))
    with pytest.raises(ValueError, match="graph_num_seqs cannot be smaller than num_seqs"):
        StepBuffers(cfg, 8, 2, "cpu").load(meta, np.array([1, 2, 3]))


def test_native_builder_pads_like_the_two_step_restatement():
    # one native pass (metadata + padding) == prepare_gen_ctx_ref followed by pad_for_graph_ref
    cfg = tiny_config()
    maxb = (cfg.max_model_len + cfg.page_size - 1) // cfg.page_size
    rng = np.random.default_rng(5)
    for n, cap_t, cap_s in ((0, 4, 2), (1, 16, 1), (3, 64, 4), (7, 128, 8)):
        reqs = []
        for s in range(n):
            done = int(rng.integers(1, cfg.max_model_len))
            this = 1 if rng.random() < 0.5 else int(rng.integers(1, min(done, 16) + 1))
            nb = (done + cfg.page_size - 1) // cfg.page_size + int(rng.integers(0, 2))
            reqs.append(dict(num_computed_tokens=done, tokens_this_step=this,
                             block_ids=rng.permutation(1000)[:min(nb, maxb)].tolist()))
        T = sum(r["tokens_this_step"] for r in reqs)
        ids = rng.integers(0, cfg.vocab_size, T)
        b = StepBuffers(cfg, cap_t, cap_s, "cpu")
        b.meta_host.fill_(0x5A)                           # stale contents must all be overwritten
        assert b.load_requests(reqs, ids, cfg.page_size) == (T, n, max([r["tokens_this_step"] for r in reqs], default=0))
        ref = OMeta.pad_for_graph_ref(OMeta.prepare_gen_ctx_ref(reqs, cfg.page_size, maxb), cap_t, cap_s)
        for k in ("slot_mapping", "positions", "context_lens", "block_tables", "query_start_loc"):
            assert np.array_equal(getattr(b, k).numpy(), ref[k]), (n, k)
        assert b.input_ids.tolist() == ids.tolist() + [0] * (cap_t - T)
        # longest context first, ties and padding in index order
        lens = ref["context_lens"]
        assert b.seq_order.tolist() == sorted(range(cap_s), key=lambda s: (-int(lens[s]), s))


def test_native_builder_rejects_inconsistent_steps():
    good = dict(num_computed_tokens=9, tokens_this_step=2, block_ids=[4, 1, 7])
    # positions 7, 8 -> block 1 row 3, block 7 row 0
    assert build_step_metadata([good], 4, 3)["slot_mapping"].tolist() == [1 * 4 + 3, 7 * 4 + 0]
    for bad in (dict(good, block_ids=[4, 1]),                    # 9 tokens need 3 blocks
                dict(good, tokens_this_step=10),                 # more new tokens than context
                dict(good, tokens_this_step=-1),
                dict(good, block_ids=[4, 1, 7, 2])):             # more blocks than a table row holds
        with pytest.raises(ValueError, match="inconsistent step"):
            build_step_metadata([bad], 4, 3)


def test_block_allocator_matches_the_scan_restatement():
    rng = np.random.default_rng(11)
    for num_blocks, page in ((1, 1), (37, 16), (500, 256)):
        cfg = types.SimpleNamespace(max_cache_blocks=num_blocks, page_size=page)
        m, ref = KC.KVCacheManager(cfg), OMeta.BlockAllocatorRef(num_blocks, page)
        held = []
        for _ in range(400):
            if held and rng.random() < 0.45:
                ids = held.pop(int(rng.integers(len(held))))
                if rng.random() < 0.3:                           # double frees and foreign ids are ignored
                    ids = ids + ids[:1] + [num_blocks + 3, -1]
                m.free_blocks(ids)
                ref.release(ids)
            else:
                tokens = int(rng.integers(0, page * max(2, num_blocks // 3)))
                cur = int(rng.integers(0, 3))
                got, want = m.allocate_blocks(tokens, cur), ref.allocate(tokens, cur)
                assert got == want, (num_blocks, tokens, cur)
                if got:
                    held.append(got)
            assert m.num_free_blocks() == len(ref.free) and m.num_allocated_blocks() == len(ref.allocated)


def test_capture_sizes_and_byte_model():
    assert capture_sizes(1) == [1]
    assert capture_sizes(5) == [1, 2, 4, 8]
    assert capture_sizes(256) == [1, 2, 4, 8, 16, 32, 64, 128, 256]
    with pytest.raises(ValueError):
        capture_sizes(0)
    cfg = qwen3_30b_a3b()
    b = decode_bytes_per_step(cfg, [1152] * 256)
    assert abs(b["moe_per_layer"] - 1.208e9) < 1e7          # 128 experts x 3 x 2048 x 768 x 2 B
    assert b["kv_per_layer"] == 256 * 1152 * 2048            # 2 x 4 kv heads x 128 x 2 B per token
    assert 88e9 < b["total"] < 92e9                          # ~60.5 GB weights + ~29 GB KV


def test_block_allocator_semantics():
    cfg = types.SimpleNamespace(max_cache_blocks=6, page_size=4)
    m = KC.KVCacheManager(cfg)
    assert m.allocate_blocks(9) == [0, 1, 2]            # lowest ids first
    assert m.allocate_blocks(9, num_current_blocks=3) == []
    assert m.allocate_blocks(13, num_current_blocks=3) == [3]
    assert m.allocate_blocks(100) is None               # out of blocks: nothing allocated
    assert m.num_free_blocks() == 2 and m.num_allocated_blocks() == 4
    m.free_blocks([1, 3, 3, 5])                          # 5 was never allocated: ignored
    assert m.num_free_blocks() == 4
    assert m.allocate_blocks(8) == [1, 3]               # freed ids are reused, lowest first
    assert m.allocate_blocks(4) == [4]


def test_kv_context_is_thread_local_and_validated():
    KC.clear_kv_cache_context()
    assert not KC.has_kv_cache_context() and KC.get_kv_cache_context() is None
    lens = torch.zeros(2, dtype=torch.int32)
    KC.set_kv_cache_context(is_paged_attn=False, context_lens=lens, query_start_loc=torch.zeros(3, dtype=torch.int32), max_seqlen_q=4)
    assert KC.has_kv_cache_context() and KC.get_kv_cache_context().max_seqlen_q == 4
    seen = []
    t = threading.Thread(target=lambda: seen.append(KC.get_kv_cache_context()))
    t.start(); t.join()
    assert seen == [None]
    with pytest.raises(AssertionError, match="key_cache required"):
        KC.set_kv_cache_context(is_paged_attn=True, context_lens=lens)
    with pytest.raises(AssertionError, match="query_start_loc required"):
        KC.set_kv_cache_context(is_paged_attn=False, context_lens=lens)
    KC.clear_kv_cache_context()


def test_kv_cache_store_shapes():
    hf = types.SimpleNamespace(num_key_value_heads=2, head_dim=8, hidden_size=64, num_attention_heads=8, num_hidden_layers=3,
                               qk_head_dim=12, v_head_dim=8)
    cc = types.SimpleNamespace(max_cache_blocks=5, page_size=4)
    st = KC.KVCacheStore(hf, cc, torch.device("cpu"))
    assert sorted(st.key_cache) == [0, 1, 2]
    assert st.key_cache[0].shape == (5, 4, 2, 12) and st.value_cache[2].shape == (5, 4, 2, 8)
    assert st.key_cache[1].dtype == torch.bfloat16 and float(st.key_cache[1].abs().sum()) == 0.0


def test_ops_refuse_cpu_tensors_and_bad_arguments():
    from vexact_amd.batch_invariant_ops import log_softmax, matmul_persistent, mean_dim, triton_bmm

    assert get_batch_invariant_attention_block_size() == AttentionBlockSize(16, 16)
    x = torch.zeros(2, 8)
    with pytest.raises(ValueError, match="only supports log_softmax along the last dimension"):
        log_softmax(x, dim=0)
    with pytest.raises(ValueError, match="must be a CUDA tensor"):
        log_softmax(x, dim=-1)
    with pytest.raises(AssertionError, match="Input must be a CUDA tensor"):
        mean_dim(x, 1)
    with pytest.raises(AssertionError, match="Incompatible dimensions"):
        matmul_persistent(torch.zeros(2, 3), torch.zeros(4, 5))
    with pytest.raises(AssertionError, match="Incompatible dtypes"):
        matmul_persistent(torch.zeros(2, 3), torch.zeros(3, 5, dtype=torch.bfloat16))
    with pytest.raises(AssertionError, match="Expected 3D tensors"):
        triton_bmm(torch.zeros(2, 3), torch.zeros(3, 5))


def test_sampler_argument_errors_need_no_gpu():
    # the reference's error cases (tests/test_inferencer_sampling.py:88-130) are raised before any device work
    from vexact_amd.inferencer.sampler import Sampler

    def cfg(**kw):
        c = types.SimpleNamespace(do_sample=True, temperature=1.0, top_k=4, top_p=1.0)
        c.__dict__.update(kw)
        return c

    s, logits = Sampler(), torch.randn(2, 16)
    with pytest.raises(ValueError, match="every request in the batch"):
        s.batch_sample_token(logits, [cfg(seed=1234), cfg()], torch.arange(2))
    with pytest.raises(ValueError, match="sampling_positions must be set"):
        s.batch_sample_token(logits, [cfg(seed=1), cfg(seed=2)])
    with pytest.raises(AssertionError, match="top_p must be set"):
        s.batch_sample_token(logits, [cfg(top_p=None)] * 2)


def test_qwen3_moe_patch_points():
    # apply_qwen3_moe_patches (vexact/models/qwen3_moe/modeling_qwen3_moe.py:291-302): idempotent, fused experts
    # container with the reference's parameter names and layout, a plain linear router
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeConfig, Qwen3MoeSparseMoeBlock

    from vexact_amd.models.qwen3_moe import (Qwen3MoeExperts, apply_qwen3_moe_patches, moe_block_forward,
                                             remove_qwen3_moe_patches)

    original = (Qwen3MoeSparseMoeBlock.__init__, Qwen3MoeSparseMoeBlock.forward)
    apply_qwen3_moe_patches()
    apply_qwen3_moe_patches()
    cfg = Qwen3MoeConfig(hidden_size=64, moe_intermediate_size=32, num_experts=8, num_experts_per_tok=2, norm_topk_prob=True,
                         num_hidden_layers=1, vocab_size=100, intermediate_size=64, num_attention_heads=2, num_key_value_heads=1)
    try:
        blk = Qwen3MoeSparseMoeBlock(cfg)
    finally:
        remove_qwen3_moe_patches()
        remove_qwen3_moe_patches()
    assert (Qwen3MoeSparseMoeBlock.__init__, Qwen3MoeSparseMoeBlock.forward) == original, "the original block is back"
    assert isinstance(blk.experts, Qwen3MoeExperts) and isinstance(blk.gate, torch.nn.Linear) and blk.gate.bias is None
    assert dict(blk.named_parameters()).keys() == {"gate.weight", "experts.gate_up_proj", "experts.down_proj"}
    assert blk.experts.gate_up_proj.shape == (8, 64, 64) and blk.experts.down_proj.shape == (8, 64, 32)
    assert (blk.top_k, blk.num_experts, blk.norm_topk_prob) == (2, 8, True)
    blk.experts = torch.nn.ModuleList()
    with pytest.raises(AssertionError, match="experts are not fused"):
        moe_block_forward(blk, torch.zeros(1, 2, 64))
    with pytest.raises(ValueError, match="silu"):
        Qwen3MoeExperts(types.SimpleNamespace(num_experts=2, hidden_size=8, moe_intermediate_size=8, hidden_act="gelu"))


def test_bench_refuses_more_than_one_gpu():
    # every pipeline stage runs on one MI355X here: asking for more must say so and exit, before any GPU work
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 2
    assert "exactly one GPU" in res.stderr and res.stdout.strip() == ""


def test_bench_hands_kernel_bench_every_option_it_reads():
    # bench.py's `configs` block runs kernel_bench.run() in-process: the arguments it builds must carry every
    # option that run() reads, or the driver's bench dies after the decode step has been measured
    import inspect
    import os
    import re
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sys.path.insert(0, root)
    import bench
    import kernel_bench

    call = re.search(r"kernel_bench\.parse\((\[.*?\])\)", inspect.getsource(bench.other_configs), re.S)
    assert call, "other_configs must build its arguments with kernel_bench.parse"
    args = kernel_bench.parse(eval(call.group(1)))
    read = set(re.findall(r"\ba\.([a-z_]+)\b", inspect.getsource(kernel_bench.run)))
    assert read and all(hasattr(args, name) for name in read), sorted(n for n in read if not hasattr(args, n))
    assert "configs" in args.what and "mfma" in args.what


def test_expert_tile_heights_and_unfilled_outputs():
    import torch

    from vexact_amd import ops

    # tile height is a function of the token count; a model that holds fragment-order expert weights only never
    # gets 128-row tiles (the one kernel that cannot read them)
    assert [ops.moe_tile_rows(t) for t in (1, 16, 17, 448, 449, 704, 705, 2047, 2048, 100000)] == [16, 16, 32, 32, 64, 64, 128, 128, 256, 256]
    assert ops.moe_tile_rows(16, packed=True) == 16 and ops.moe_tile_rows(3, top_k=2, num_experts=16) == 16
    assert [ops.moe_tile_rows(t, packed_only=True) for t in (256, 448, 449, 832, 833, 2048)] == [32, 32, 64, 64, 256, 256]
    assert [ops.moe_tile_rows(t, packed=True) for t in (256, 448, 449, 832, 833, 2048)] == [32, 32, 64, 64, 256, 256]
    assert ops.moe_tile_rows(5000, wide_ok=False) == 128 and ops.moe_tile_rows(5000, wide_ok=False, packed_only=True) == 64
    # keyed on the rows an average expert receives, not on the token count: 256 experts / top-8 reach a tile height at
    # twice the tokens, 16 experts / top-2 at half of them (4096 tokens x 2 / 16 = 512 rows per expert = 8192 tokens of
    # the measured 128-expert / top-8 shape)
    assert [ops.moe_tile_rows(t, num_experts=256) for t in (896, 898, 1408, 1410, 4095, 4096)] == [32, 64, 64, 128, 128, 256]
    assert [ops.moe_tile_rows(t, top_k=2, num_experts=16) for t in (224, 225, 352, 353, 1023, 1024)] == [32, 64, 64, 128, 128, 256]
    assert [ops.moe_tile_rows(t, packed=True, top_k=2, num_experts=16) for t in (224, 225, 416, 417)] == [32, 64, 64, 256]
    assert ops.moe_tile_rows(4096, top_k=1, num_experts=1) == 256 and ops.moe_tile_rows(20, top_k=1, num_experts=1) == 32
    # outputs that a kernel overwrites completely skip the NaN fill of deterministic mode and leave the switch as it was
    was = torch.are_deterministic_algorithms_enabled()
    try:
        torch.use_deterministic_algorithms(True)
        assert torch.utils.deterministic.fill_uninitialized_memory
        assert bool(torch.empty(64).isnan().all())
        t = ops._empty((3, 5), dtype=torch.float32, device="cpu")
        assert t.shape == (3, 5) and torch.utils.deterministic.fill_uninitialized_memory
        assert ops._empty_like(torch.zeros(4, dtype=torch.bfloat16)).dtype == torch.bfloat16
        torch.utils.deterministic.fill_uninitialized_memory = False
        ops._empty(2, dtype=torch.float32, device="cpu")
        assert not torch.utils.deterministic.fill_uninitialized_memory
    finally:
        torch.utils.deterministic.fill_uninitialized_memory = True
        torch.use_deterministic_algorithms(was)



def test_gemm_piece_addresses_below_the_step_width_stay_inside_the_row():
    # The weight-streaming GEMM loads, per lane group g = 0..3 and unrolled slot u, the 16-byte piece at element
    # kstep0 + 32 u + 8 g of a row of K elements (K a multiple of 8); a piece past K is replaced by the row's first
    # piece (offset -8 g from the lane's base pointer, which already points 8 g into the row) and zeroed. The tiled
    # kernel does the same with 64-wide steps and piece index c8 = 0..7. Every address touched must lie inside the row.
    def offsets_stream(K, U):
        out = []
        for kstep0 in range(0, K, 32 * U):
            for u in range(U):
                for g in range(4):
                    ok = kstep0 + 32 * u + 8 * g < K
                    out.append(8 * g + (kstep0 + 32 * u if ok else -8 * g))   # lane base + offset
        return out

    def offsets_tiled(K):
        out = []
        for k0 in range(0, K, 64):
            for c8 in range(8):
                ok = k0 + 8 * c8 < K
                out.append(8 * c8 + (k0 if ok else -8 * c8))
        return out

    for K in (8, 16, 24, 32, 40, 56, 64, 72, 200):
        for U in (1, 2, 4, 8):
            assert all(0 <= o <= K - 8 for o in offsets_stream(K, U)), (K, U)
        assert all(0 <= o <= K - 8 for o in offsets_tiled(K)), K


def test_fragment_order_image_holds_whole_load_groups():
    # The streaming kernel reads a fragment-order weight image in groups of 8 k-chunks (32 k-elements each) without
    # any mask: the image must therefore be zero-filled to a multiple of 8 chunks that covers K, or the last group of
    # a row block would run into the next block (past the tensor for the last block of the last expert).
    from vexact_amd import _lib
    lib = _lib.load()
    for K in list(range(1, 600)) + [767, 768, 769, 2047, 2048, 2049, 4096, 12288]:
        ch = lib.vx_packed_kchunks(K)
        assert ch % 8 == 0 and 32 * ch >= K and 32 * (ch - 8) < K, (K, ch)


def test_host_metadata_and_allocator_under_address_and_ub_sanitizers():
    # the native step-metadata builder and block allocator on 400 random steps and 50 random allocate / free traces with
    # exactly sized heap buffers, compiled with -fsanitize=address,undefined: an access outside a buffer aborts the run
    import os
    import subprocess
    import tempfile
    here = os.path.dirname(os.path.abspath(__file__))
    with tempfile.TemporaryDirectory() as d:
        exe = os.path.join(d, "host_meta_sanitized")
        subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                        "-static-libasan", "-o", exe, os.path.join(here, "host_meta_sanitized.cpp")], check=True)
        run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "sanitized run ok" in run.stdout


def test_attention_row_block_numbering_covers_every_block_once(tmp_path):
    """Which (sequence, row block, head group) a workgroup of the general attention kernels works on is decided by two pieces
    of plain C++ in vexact_amd/csrc/attn_core.h: the host lambda that sizes the grid (plain or compact numbering) and the
    device function locate_row_block. Both are compiled here for the host from the source text, unchanged, and every workgroup
    of the grid is walked: each block that holds query rows must be reached exactly once, in every form."""
    import ctypes
    import os
    import subprocess

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "vexact_amd", "csrc", "attn_core.h")).read()
    a = text.index("__device__ __forceinline__ bool locate_row_block(")
    locate = text[a:text.index("__device__ __forceinline__ float fast_exp2", a)]
    b = text.index("    auto row_grid = [&](int rb, unsigned heads) {")
    row_grid = text[b:text.index("    dim3 grid = row_grid(", b)]
    src = tmp_path / "row_blocks.cpp"
    src.write_text(
        "#include <algorithm>\n#include <stdint.h>\n#define __device__\n#define __forceinline__ inline\n"
        "struct dim3 { unsigned x, y, z; dim3(unsigned a = 1, unsigned b = 1, unsigned c = 1) : x(a), y(b), z(c) {} };\n"
        "struct AttnParams { const int* cu_q; int num_seqs, compact, grid_heads, grid_sg; };\n"
        "static dim3 blockIdx, gridDim;\n" + locate +
        'extern "C" int walk(const int* cu_q, int num_seqs, int total_q, int max_q, int rpb, unsigned nheads, int* counts, int maxblocks,\n'
        "                    int* form) {\n"
        "  AttnParams p = {cu_q, num_seqs, 0, 0, 0};\n"
        "  const int rows = max_q > 0 ? max_q : total_q;\n" + row_grid +
        "  const dim3 grid = row_grid(rpb, nheads);\n"
        "  gridDim = grid;\n  *form = p.compact;\n  int stray = 0;\n"
        "  for (unsigned z = 0; z < grid.z; z++) for (unsigned y = 0; y < grid.y; y++) for (unsigned x = 0; x < grid.x; x++) {\n"
        "    blockIdx = dim3(x, y, z);\n    int seq, bx, hg;\n"
        "    if (!locate_row_block(p, rpb, seq, bx, hg)) continue;\n"
        "    if (seq < 0 || seq >= num_seqs || hg < 0 || hg >= (int)nheads || bx < 0) { stray++; continue; }\n"
        "    if ((int64_t)bx * rpb >= cu_q[seq + 1] - cu_q[seq]) continue;  // no query row in this block: the kernel leaves at once\n"
        "    if (bx >= maxblocks) { stray++; continue; }\n"
        "    counts[((int64_t)seq * maxblocks + bx) * nheads + hg]++;\n  }\n  return stray;\n}\n")
    so = tmp_path / "row_blocks.so"
    subprocess.run(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-o", str(so), str(src)], check=True)
    lib = ctypes.CDLL(str(so))
    rng = np.random.default_rng(11)
    forms = set()
    batches = [[512] * 4, [1] * 40 + [700], [1, 1, 8192, 1], [0, 5, 0, 0, 33], [70000], [3] * 300, [2048, 1, 1, 1, 1, 1, 1, 1, 900]]
    batches += [list(rng.integers(0, 300, rng.integers(1, 12))) for _ in range(20)]
    batches.append([1_100_000, 3])  # more row blocks of 16 than a grid dimension can count
    for lens in batches:
        if sum(lens) == 0:
            continue
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        huge = sum(lens) > 1_000_000
        for rpb in ((16,) if huge else (16, 32, 64, 128, 256)):
            for nheads in ((2,) if huge else (1, 2, 4, 8, 32)):
                for max_q in (int(max(lens)), 0):  # 0 = unknown: the launch then assumes total_q rows per sequence
                    maxblocks = int((max(lens) + rpb - 1) // rpb)
                    counts = np.zeros((len(lens), maxblocks, nheads), dtype=np.int32)
                    form = ctypes.c_int(-1)
                    stray = lib.walk(cu.ctypes.data_as(ctypes.c_void_p), len(lens), int(sum(lens)), int(max_q), rpb, nheads,
                                     counts.ctypes.data_as(ctypes.c_void_p), maxblocks, ctypes.byref(form))
                    forms.add(form.value)
                    assert stray == 0, (lens, rpb, nheads, max_q)
                    want = np.zeros_like(counts)
                    for s, n in enumerate(lens):
                        want[s, : (n + rpb - 1) // rpb, :] = 1
                    assert np.array_equal(counts, want), (lens, rpb, nheads, max_q, form.value)
    assert forms == {0, 1, 2}, forms  # the plain grid, the compact numbering, and its form for more than 65535 items


def test_wide_gemm_tile_walk_reaches_every_tile_once(tmp_path):
    """The persistent 256 x 256 GEMM kernel hands tiles out by a fixed rule: workgroup b of G starts at
    (b & 7) (G / 8) + (b >> 3) and steps by G, and tile number -> (rows, columns) goes through tile_at (groups of four row
    tiles for the dense form, the expert tile table for the grouped one). That text of vexact_amd/csrc/gemm_wide.h is compiled
    here for the host, unchanged: over all workgroups every output tile must come up exactly once."""
    import ctypes
    import os
    import subprocess

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "vexact_amd", "csrc", "gemm_wide.h")).read()
    a = text.index("  const int G = gridDim.x;  // multiple of 8")
    walk = text[a:text.index("  if (first >= tiles || !tile_at(first).ok) return;", a)]
    group_m = int(text.split("constexpr int WD_GROUP_M = ")[1].split(";")[0])

    def variant(name, grouped):
        body = walk.replace("if constexpr (GROUPED)", "if constexpr (%s)" % ("true" if grouped else "false"))
        return ("extern \"C\" int @NAME@(int M, int tiles_m, int tiles_n, int G_, const int* tg, const int* tr0, const int* trows, int BM, int NOUT,\n"
                "                int* out /* [tiles][4]: row0, rows, n0, ok */, int* hits) {\n"
                "  struct { int M; const int* tile_group; const int* tile_row0; const int* tile_rows; int64_t w_gstride; } p = {M, tg, tr0, trows, 1000};\n"
                "  const int tiles = tiles_m * tiles_n;\n  struct { unsigned x; } gridDim = {(unsigned)G_}, blockIdx = {0};\n"
                "  for (unsigned b = 0; b < (unsigned)G_; b++) {\n    blockIdx.x = b;\n" + body +
                "    for (int lin = first; lin < tiles; lin += G) {\n      const WideTile t = tile_at(lin);\n"
                "      out[4 * lin] = t.row0; out[4 * lin + 1] = t.rows; out[4 * lin + 2] = t.n0; out[4 * lin + 3] = t.ok; hits[lin]++;\n"
                "    }\n  }\n  return 0;\n}\n").replace("@NAME@", name)

    src = tmp_path / "tile_walk.cpp"
    src.write_text("#include <algorithm>\n#include <stdint.h>\nusing std::min;\nconstexpr int WD_GROUP_M = %d;\n"
                   "struct WideTile { int row0, rows, n0; int64_t wbase; bool ok; };\n" % group_m
                   + variant("walk_dense", False) + variant("walk_grouped", True))
    so = tmp_path / "tile_walk.so"
    subprocess.run(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-o", str(so), str(src)], check=True)
    lib = ctypes.CDLL(str(so))
    P = lambda x: x.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    rng = np.random.default_rng(3)
    for BM, NOUT in ((256, 256), (128, 256), (256, 128)):
        for M, N in ((8192, 5120), (300, 256), (4097, 1000), (256 * 7 + 1, 151936), (100, 100)):
            tiles_m, tiles_n = (M + BM - 1) // BM, (N + NOUT - 1) // NOUT
            for G in (8, 64, 256):
                out = np.full((tiles_m * tiles_n, 4), -1, dtype=np.int32)
                hits = np.zeros(tiles_m * tiles_n, dtype=np.int32)
                lib.walk_dense(M, tiles_m, tiles_n, G, None, None, None, BM, NOUT, P(out), P(hits))
                assert (hits == 1).all(), (M, N, BM, G)
                seen = {(int(r), int(c)) for r, _, c, _ in out}
                assert seen == {(i * BM, j * NOUT) for i in range(tiles_m) for j in range(tiles_n)}
                assert all(int(rows) == min(BM, M - int(r0)) and ok == 1 for r0, rows, _, ok in out)
    # grouped: a table of row tiles (expert, first row, rows), unused entries marked -1 at the end
    for _ in range(20):
        n_tiles, spare, tiles_n, G = int(rng.integers(1, 400)), int(rng.integers(0, 9)), int(rng.integers(1, 9)), int(rng.choice([8, 64, 256]))
        tg = np.concatenate([np.sort(rng.integers(0, 128, n_tiles)), -np.ones(spare)]).astype(np.int32)
        tr0 = np.concatenate([np.arange(n_tiles) * 256, np.zeros(spare)]).astype(np.int32)
        trows = np.concatenate([rng.integers(1, 257, n_tiles), np.zeros(spare)]).astype(np.int32)
        tiles_m = n_tiles + spare
        out = np.full((tiles_m * tiles_n, 4), -1, dtype=np.int32)
        hits = np.zeros(tiles_m * tiles_n, dtype=np.int32)
        lib.walk_grouped(0, tiles_m, tiles_n, G, P(tg), P(tr0), P(trows), 256, 256, P(out), P(hits))
        assert (hits == 1).all()
        real = out[out[:, 3] == 1]
        assert {(int(r), int(c)) for r, _, c, _ in real} == {(int(r), j * 256) for r in tr0[:n_tiles] for j in range(tiles_n)}
        assert len(real) == n_tiles * tiles_n and (out[out[:, 3] == 0].shape[0] == spare * tiles_n)


def test_paged_key_addresses_stay_inside_the_sequence_pages(tmp_path):
    """Where the attention kernels read a sequence's keys and values is decided by KVSource in
    vexact_amd/csrc/attn_core.h (page lookup per 16-key tile for power-of-two pages, per key otherwise, packed rows without a
    table). Its text is compiled for the host with -fsanitize=address and driven the way the kernels drive it (64-key blocks,
    lanes past the end asking for row 0 of their tile): the block-table row is an exactly sized heap array holding only the
    sequence's own pages, so a lookup past them aborts, and every address must be the row of an existing key (the right one
    for keys below the length)."""
    import os
    import subprocess

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "vexact_amd", "csrc", "attn_core.h")).read()
    a = text.index("enum : int { SRC_FAST = 0, SRC_GENERIC = 1, SRC_PACKED = 2 };")
    b = text.index("template <int KIND>\nstruct KVSource {", a)
    struct = text[a:text.index("\n};\n", b) + 4]
    src = tmp_path / "kv_source.cpp"
    src.write_text(
        "#include <algorithm>\n#include <cstdio>\n#include <cstdlib>\n#include <random>\n#include <stdint.h>\n#include <vector>\n"
        "#define __device__\n#define __forceinline__ inline\nusing std::min;\ntypedef uint16_t bf16_t;\n" + struct + r"""
#define CHECK(c) do { if (!(c)) { std::fprintf(stderr, "check failed at line %d: %s\n", __LINE__, #c); std::exit(1); } } while (0)
template <int KIND>
static void run(std::mt19937_64& rng) {
  auto rnd = [&](int64_t lo, int64_t hi) { return lo + (int64_t)(rng() % (uint64_t)(hi - lo + 1)); };
  for (int it = 0; it < 300; it++) {
    const int ps = KIND == SRC_FAST ? (16 << rnd(0, 4)) : (int)rnd(1, 40);
    const int kv_len = (int)rnd(1, 700), npages = (kv_len + ps - 1) / ps, pool = npages + (int)rnd(0, 50);
    std::vector<int> table((size_t)npages);  // exactly the sequence's pages: a lookup past them is a heap overflow
    for (auto& t : table) t = (int)rnd(0, pool - 1);
    const int64_t D = 128, skp = 4 * D, skb = (int64_t)ps * skp;  // [blocks, page, 4 heads, D]
    KVSource<KIND> s;
    s.kbase = (const bf16_t*)0 + 2 * D; s.vbase = (const bf16_t*)0 + 3 * D;  // kv heads 2 and 3; offsets only, never dereferenced
    s.bt = KIND == SRC_PACKED ? nullptr : table.data();
    s.skb = skb; s.skp = skp; s.svb = skb; s.svp = skp;
    s.ps = ps; s.last = kv_len - 1;
    s.shift = -1;
    if ((ps & (ps - 1)) == 0) { s.shift = 0; while ((1 << s.shift) < ps) s.shift++; }
    if (KIND == SRC_GENERIC && rnd(0, 1)) s.shift = -1;  // the division form also for power-of-two pages
    for (int kb = 0; kb < kv_len; kb += 64) {
      const typename KVSource<KIND>::Tiles tl = s.tiles(kb);
      for (int tt = 0; tt < 4; tt++)
        for (int lane_row = 0; lane_row < 16; lane_row++) {
          const int key = kb + 16 * tt + lane_row;
          const bool ok = key < kv_len;
          const int within = ok ? lane_row : 0;  // what issue_k / issue_v pass
          for (int is_v = 0; is_v < 2; is_v++) {
            const bf16_t* r = is_v ? s.vrow(tl, kb, tt, within) : s.krow(tl, kb, tt, within);
            const int64_t off = (r - (const bf16_t*)0) - (is_v ? 3 : 2) * D;
            CHECK(off >= 0 && off % skp == 0);
            const int64_t row = off / skp;
            if (KIND == SRC_PACKED) {
              CHECK(row == (ok ? key : std::min(kb + 16 * tt, kv_len - 1)));
            } else {
              const int64_t page = row / ps, in_page = row % ps;
              bool found = false;  // the row of an existing key of this sequence
              for (int pg = 0; pg < npages && !found; pg++) found = table[(size_t)pg] == page && pg * ps + in_page < kv_len;
              CHECK(found);
              if (ok) CHECK(page == table[(size_t)(key / ps)] && in_page == key % ps);
            }
          }
        }
    }
  }
}
int main() {
  std::mt19937_64 rng(99);
  run<SRC_FAST>(rng);
  run<SRC_GENERIC>(rng);
  run<SRC_PACKED>(rng);
  std::puts("kv source sanitized run ok");
  return 0;
}
""")
    exe = tmp_path / "kv_source"
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-static-libasan",
                    "-o", str(exe), str(src)], check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "sanitized run ok" in run.stdout


def test_tile_table_bound_holds_for_any_split_of_the_rows():
    # vx_moe_max_tiles(n, E, bm) sizes the tile table that the routing kernel fills with ceil(rows_e / bm) tiles per expert:
    # it must be an upper bound for every way n (token, slot) entries can fall on E experts, and it is attained.
    from vexact_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(2)
    for _ in range(3000):
        E, bm = int(rng.integers(1, 300)), int(rng.choice([16, 32, 64, 128, 256]))
        n = int(rng.integers(0, 5000))
        kind = rng.integers(0, 3)
        if kind == 0:      # uniform
            rows = np.bincount(rng.integers(0, E, n), minlength=E)
        elif kind == 1:    # everything on a few experts
            rows = np.bincount(rng.integers(0, min(E, 3), n), minlength=E)
        else:              # as many experts as possible one past a multiple of the tile height
            rows = np.zeros(E, dtype=np.int64)
            left = n
            for e in range(E):
                take = min(left, bm * int(rng.integers(0, 3)) + 1)
                rows[e], left = take, left - take
            rows[0] += left
        tiles = int(((rows + bm - 1) // bm).sum())
        assert tiles <= lib.vx_moe_max_tiles(n, E, bm), (n, E, bm, tiles)
    # attained: min(E, n) experts with one row beyond whole tiles
    assert lib.vx_moe_max_tiles(3 * 32 + 3, 3, 32) == 3 + 3 and int(((np.array([33, 33, 33]) + 31) // 32).sum()) == 6
