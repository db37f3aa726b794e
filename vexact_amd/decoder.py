"""A Qwen3-MoE-shaped decoder that runs entirely on the HIP kernels, with paged KV, bucketed
static buffers and HIP-graph capture of the decode step.

It plays the part of the reference's model runner for this architecture:
``Inferencer._prepare_gen_ctx`` / ``_prepare_input_buffers_from_gen_ctx``
(vexact/inferencer/inferencer.py:193-349: integer metadata and the padding rules of a captured
bucket), ``CudaGraphManager`` (vexact/inferencer/cudagraph_utils.py:45-190: power-of-two token
buckets, capture, padded replay) and ``_select_tokens`` (inferencer.py:391-449: last-token gather,
greedy token, fp32 logprob). The layer itself follows the HuggingFace Qwen3-MoE decoder layer the
reference patches (RMSNorm -> q/k/v -> per-head q/k norm -> rotary -> paged attention -> o_proj ->
residual -> RMSNorm -> router -> fused experts -> residual), all pipeline stages on one device.
"""

from __future__ import annotations

import ctypes
import itertools
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np
import torch

from . import ops


@dataclass
class DecoderConfig:
    hidden_size: int = 2048
    num_layers: int = 48
    num_heads: int = 32
    num_kv_heads: int = 4
    head_dim: int = 128
    num_experts: int = 128
    top_k: int = 8
    moe_intermediate: int = 768
    vocab_size: int = 151936
    rms_eps: float = 1e-6
    rope_theta: float = 1.0e6
    norm_topk_prob: bool = True
    page_size: int = 16
    max_model_len: int = 4096

    @property
    def qkv_dim(self) -> int:
        return (self.num_heads + 2 * self.num_kv_heads) * self.head_dim


def qwen3_30b_a3b() -> DecoderConfig:
    return DecoderConfig()


def tiny_config(**kw) -> DecoderConfig:
    base = dict(hidden_size=256, num_layers=2, num_heads=4, num_kv_heads=2, head_dim=128, num_experts=8, top_k=2,
                moe_intermediate=128, vocab_size=1000, max_model_len=512)
    base.update(kw)
    return DecoderConfig(**base)


class DecoderWeights:
    """bf16 weights; q/k/v projections are stored fused as one ``[(Hq+2Hkv)*D, H]`` matrix and the
    expert gate/up projections as ``[E, 2I, H]`` (gate rows first), like the reference's
    ``Qwen3MoeExperts`` (vexact/models/qwen3_moe/modeling_qwen3_moe.py:42-67)."""

    def __init__(self, cfg: DecoderConfig, device="cuda", seed: int = 5, std: float = 0.02, generator_device="cuda",
                 norm_std: float = 0.0):
        """``norm_std``: spread of the RMSNorm weights around 1 (0 = exactly 1, a freshly initialised model)."""
        self.cfg = cfg
        g = torch.Generator(device=generator_device).manual_seed(seed)
        bf = torch.bfloat16

        def rnd(*shape):
            t = torch.empty(shape, dtype=bf, device=generator_device)
            t.normal_(0.0, std, generator=g)
            return t.to(device)

        def rnd_pitched(*shape):
            # Rows whose pitch is a multiple of 2 KB land on few HBM channels when 16 of them are
            # streamed side by side; 128 bytes of padding per row spread them (about 4 % on the
            # expert gate/up GEMM). The tensor handed out is the [..., :K] view of the padded buffer.
            t = rnd(*shape)
            if (shape[-1] * 2) % 2048 != 0:
                return t
            buf = torch.empty(*shape[:-1], shape[-1] + 64, dtype=bf, device=device)
            buf[..., : shape[-1]] = t
            return buf[..., : shape[-1]]

        H, D, E, I = cfg.hidden_size, cfg.head_dim, cfg.num_experts, cfg.moe_intermediate
        def ones(n):
            if norm_std == 0.0:
                return torch.ones(n, dtype=bf, device=device)
            t = torch.empty(n, dtype=torch.float32, device=generator_device)
            t.normal_(1.0, norm_std, generator=g)
            return t.to(bf).to(device)

        self.embed = rnd(cfg.vocab_size, H)
        self.lm_head = rnd(cfg.vocab_size, H)
        self.final_norm = ones(H)
        self.layers = []
        for _ in range(cfg.num_layers):
            self.layers.append(
                dict(
                    in_norm=ones(H),
                    qkv=rnd(cfg.qkv_dim, H),
                    q_norm=ones(D),
                    k_norm=ones(D),
                    o=rnd(H, cfg.num_heads * D),
                    post_norm=ones(H),
                    router=rnd(E, H),
                    gate_up=rnd_pitched(E, 2 * I, H),
                    down=rnd(E, H, I),
                )
            )

        self.packed = None
        self.packed_only = False

    def pack_experts(self, keep_unpacked: bool = True, low_peak: bool = False) -> None:
        """Add fragment-order copies of the expert weights (``ops.pack_expert_weights``). Steps whose expert
        tiles have at most 64 rows (decode) stream them, and so do 256-row tiles (prefill chunks); only the
        128-row kernel needs the ``[E, N, K]`` tensors. ``keep_unpacked=False`` frees those tensors, so that the
        model holds one copy of its expert weights (the decoder then never picks 128-row tiles; call this before
        the first ``bucket()``); weights are then updated by loading new ``[E, N, K]`` tensors into ``layers[i]``
        and packing again. By default every layer is packed before anything is freed and the freed memory goes
        back to the driver, so both copies exist for a moment; ``low_peak=True`` frees layer by layer instead
        (the packed tensors then land in recycled blocks, measured 1.5 % slower per decode step). With
        ``keep_unpacked=True`` call this again, or ``invalidate_packed()``, after the weights change."""
        if self.packed_only:
            raise RuntimeError("the [E, N, K] expert tensors have been freed: nothing to pack from")
        self.packed = []
        for l in self.layers:
            self.packed.append((ops.pack_expert_weights(l["gate_up"]), ops.pack_expert_weights(l["down"])))
            if not keep_unpacked and low_peak:
                l["gate_up"] = l["down"] = None
        if not keep_unpacked:
            for l in self.layers:
                l["gate_up"] = l["down"] = None
            torch.cuda.empty_cache()  # hand the freed tensors' memory back, so that later allocations start afresh
        self.packed_only = not keep_unpacked

    def invalidate_packed(self) -> None:
        """Drop the fragment-order copies. They are plain copies that nothing tracks: after any write to
        ``layers[i]["gate_up"]`` / ``["down"]`` call this (decode then streams the ``[E, N, K]`` tensors again)
        or ``pack_experts()``; a decode graph captured earlier still replays the old copies and has to be
        captured again."""
        if self.packed_only:
            raise RuntimeError("the fragment-order copies are the only expert weights left")
        self.packed = None

    def nbytes(self) -> int:
        """Bytes of the model's weights (one copy of each; fragment-order copies kept beside ``[E, N, K]`` tensors
        are extra)."""
        n = self.embed.numel() + self.lm_head.numel() + self.final_norm.numel()
        for l in self.layers:
            n += sum(t.numel() for t in l.values() if t is not None)
        if self.packed_only:
            n += sum(a.data.numel() + b.data.numel() for a, b in self.packed)
        return 2 * n

    def to_cpu(self) -> "DecoderWeights":
        c = object.__new__(DecoderWeights)
        c.cfg = self.cfg
        c.embed, c.lm_head, c.final_norm = self.embed.cpu(), self.lm_head.cpu(), self.final_norm.cpu()
        if self.packed_only:
            raise RuntimeError("the [E, N, K] expert tensors have been freed")
        c.layers = [{k: v.cpu() for k, v in l.items()} for l in self.layers]
        c.packed = None
        c.packed_only = False
        return c


def rope_tables(cfg: DecoderConfig, device) -> tuple[torch.Tensor, torch.Tensor]:
    """cos / sin ``[max_model_len, D]`` in bf16: fp32 ``position * inv_freq`` duplicated over both
    halves, then cast (what HuggingFace's rotary embedding yields for bf16 activations)."""
    D = cfg.head_dim
    inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    pos = torch.arange(cfg.max_model_len, dtype=torch.float32)
    freqs = pos[:, None] * inv_freq[None, :]
    emb = torch.cat([freqs, freqs], dim=-1)
    return emb.cos().to(torch.bfloat16).to(device), emb.sin().to(torch.bfloat16).to(device)


def _flatten_requests(requests: Sequence[dict]):
    """``requests`` hold ``num_computed_tokens`` (after this step), ``tokens_this_step`` and
    ``block_ids``; returns the flat int arrays the native builder reads."""
    B = len(requests)
    done = np.fromiter((r["num_computed_tokens"] for r in requests), np.int64, B)
    n_tok = np.fromiter((r["tokens_this_step"] for r in requests), np.int64, B)
    offs = np.zeros(B + 1, np.int64)
    np.cumsum(np.fromiter((len(r["block_ids"]) for r in requests), np.int64, B), out=offs[1:])
    if B and all(isinstance(r["block_ids"], np.ndarray) for r in requests):  # the fast form: no per-id Python work
        ids = np.concatenate([r["block_ids"] for r in requests]).astype(np.int32, copy=False)
    else:
        ids = np.fromiter(itertools.chain.from_iterable(r["block_ids"] for r in requests), np.int32, int(offs[-1]))
    return done, n_tok, ids, offs


def _native_step_metadata(requests, page_size, max_blocks, cap_tokens, cap_seqs, positions, slot, qsl, lens, bt, order=None):
    """One call of ``vx_host_step_metadata`` writing into the given host addresses (ints)."""
    from . import _lib

    done, n_tok, ids, offs = _flatten_requests(requests)
    total, maxq = ctypes.c_int64(0), ctypes.c_int32(0)
    rc = _lib.load().vx_host_step_metadata(
        len(requests), done.ctypes.data, n_tok.ctypes.data, ids.ctypes.data, offs.ctypes.data, page_size, max_blocks,
        cap_tokens, cap_seqs, positions, slot, qsl, lens, bt, order, ctypes.byref(total), ctypes.byref(maxq))
    if rc != 0:
        # say which of the reference's conditions failed (inferencer.py:306-311), else the generic message
        if len(requests) > cap_seqs:
            raise ValueError(f"graph_num_seqs cannot be smaller than num_seqs: {cap_seqs} < {len(requests)}")
        if int(n_tok.sum()) > cap_tokens:
            raise ValueError(f"total_tokens exceeds capture_tokens: {int(n_tok.sum())} > {cap_tokens}")
        raise ValueError("inconsistent step: a request's token counts or block ids do not cover its context, "
                         f"or it holds more than {max_blocks} blocks")
    return total.value, maxq.value


def build_step_metadata(requests: Sequence[dict], page_size: int, max_blocks_per_req: int) -> dict:
    """Integer metadata of one step at its exact size (no bucket padding), built by the native
    host routine. ``requests`` hold ``num_computed_tokens`` (after this step), ``tokens_this_step``
    and ``block_ids``."""
    B = len(requests)
    T = int(sum(max(0, r["tokens_this_step"]) for r in requests))
    positions, slot = np.empty(T, np.int64), np.empty(T, np.int32)
    qsl, lens = np.empty(B + 1, np.int32), np.empty(B, np.int32)
    bt = np.empty((B, max_blocks_per_req), np.int32)
    _, maxq = _native_step_metadata(requests, page_size, max_blocks_per_req, T, B, positions.ctypes.data, slot.ctypes.data,
                                    qsl.ctypes.data, lens.ctypes.data, bt.ctypes.data)
    return {
        "slot_mapping": slot,
        "context_lens": lens,
        "block_tables": bt,
        "query_start_loc": qsl,
        "max_seqlen_q": maxq,
        "positions": positions,
    }


def capture_sizes(max_size: int) -> list[int]:
    """1, 2, 4, ... up to the first power of two >= max_size (cudagraph_utils.py:84-94)."""
    if max_size <= 0:
        raise ValueError(f"max_size must be positive or None, got {max_size}")
    sizes, s = [], 1
    while s < max_size:
        sizes.append(s)
        s *= 2
    sizes.append(s)
    return sizes


class StepBuffers:
    """Static device buffers of one (num_tokens, num_seqs) bucket."""

    def __init__(self, cfg: DecoderConfig, num_tokens: int, num_seqs: int, device, packed_only: bool = False,
                 packed: bool = False):
        """``packed_only``: the model holds fragment-order expert weights only (no 128-row expert tiles)."""
        T, B = num_tokens, num_seqs
        self.num_tokens, self.num_seqs = T, B
        self.max_blocks = (cfg.max_model_len + cfg.page_size - 1) // cfg.page_size
        i32, i64, bf = torch.int32, torch.int64, torch.bfloat16
        z = lambda *s, dtype: torch.zeros(s, dtype=dtype, device=device)  # noqa: E731
        # All integer metadata lives in ONE device allocation mirrored by one (pinned) host staging
        # buffer with the same layout, so that a step costs one host-to-device copy.
        mb = self.max_blocks
        segs = (("positions", i64, (T,)), ("input_ids", i64, (T,)), ("slot_mapping", i32, (T,)),
                ("query_start_loc", i32, (B + 1,)), ("context_lens", i32, (B,)), ("seq_order", i32, (B,)),
                ("block_tables", i32, (B, mb)))
        offs, end = {}, 0
        for name, dt, shape in segs:
            offs[name] = end
            end += -(-int(np.prod(shape)) * (8 if dt == i64 else 4) // 64) * 64
        on_gpu = torch.device(device).type == "cuda"
        self.meta_dev = torch.zeros(end, dtype=torch.uint8, device=device)
        self.meta_host = torch.zeros(end, dtype=torch.uint8, pin_memory=on_gpu)
        self._host = {}
        for name, dt, shape in segs:
            n = int(np.prod(shape)) * (8 if dt == i64 else 4)
            setattr(self, name, self.meta_dev[offs[name]: offs[name] + n].view(dt).view(shape))
            self._host[name] = self.meta_host[offs[name]: offs[name] + n].view(dt).view(shape).numpy()
        self._host_ptr = {k: v.ctypes.data for k, v in self._host.items()}
        self._host["slot_mapping"].fill(-1)
        self._host["block_tables"].fill(-1)
        self._host["seq_order"][:] = np.arange(B)
        self.meta_dev.copy_(self.meta_host)
        H, k = cfg.hidden_size, cfg.top_k
        self.x = z(T, H, dtype=bf)
        self.h = z(T, H, dtype=bf)
        self.qkv = z(T, cfg.qkv_dim, dtype=bf)
        self.q = z(T, cfg.num_heads, cfg.head_dim, dtype=bf)
        self.attn = z(T, cfg.num_heads, cfg.head_dim, dtype=bf)
        self.o = z(T, H, dtype=bf)
        self.router_logits = z(T, cfg.num_experts, dtype=bf)
        self.topk_w = z(T, k, dtype=bf)
        self.topk_idx = z(T, k, dtype=i32)
        self.hw = z(T * k, cfg.moe_intermediate, dtype=bf)
        self.eo = z(T * k, H, dtype=bf)
        self.bm = ops.moe_tile_rows(T, wide_ok=(cfg.hidden_size % 64 == 0 and cfg.moe_intermediate % 64 == 0),
                                    packed_only=packed_only, packed=packed, top_k=k, num_experts=cfg.num_experts)
        from . import _lib

        lib = _lib.load()
        self.max_tiles = lib.vx_moe_max_tiles(T * k, cfg.num_experts, self.bm)
        self.route_ints = z(2 * cfg.num_experts + 1 + 3 * T * k + 3 * self.max_tiles, dtype=i32)
        # chunk states of the split decode form (nothing when this bucket's decode takes the fused form)
        self.attn_ws_bytes = lib.vx_paged_attn_decode_workspace_needed(B, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim,
                                                                      self.max_blocks * cfg.page_size, 0)
        self.attn_ws = None  # handed out by the decoder: one workspace shared by all buckets
        # sampling: one row per sequence
        self.last_h = z(B, H, dtype=bf)
        self.logits = z(B, cfg.vocab_size, dtype=bf)
        self.logprobs = z(B, dtype=torch.float32)
        self.tokens = z(B, dtype=i64)
        self.seeds = z(B, dtype=i64)       # per-sequence sampling seeds (set by the caller)
        self.sample_pos = z(B, dtype=i64)  # position of the token being sampled = context length

    def load(self, meta: dict, input_ids: np.ndarray) -> tuple[int, int]:
        """Copy one step's metadata in, applying the bucket padding rules (inferencer.py:306-324):
        pad tokens get id 0, position 0, slot -1; pad sequences get ``query_start_loc = T_real``,
        ``context_len = 0`` and an all-zero block-table row."""
        T, B = len(input_ids), len(meta["context_lens"])
        if T > self.num_tokens:
            raise ValueError(f"total_tokens exceeds capture_tokens: {T} > {self.num_tokens}")
        if B > self.num_seqs:
            raise ValueError(f"graph_num_seqs cannot be smaller than num_seqs: {self.num_seqs} < {B}")
        h = self._host
        h["positions"][:T] = meta["positions"]; h["positions"][T:] = 0
        h["slot_mapping"][:T] = meta["slot_mapping"]; h["slot_mapping"][T:] = -1
        w = min(meta["block_tables"].shape[1], self.max_blocks)
        h["block_tables"][:B] = -1; h["block_tables"][B:] = 0
        h["block_tables"][:B, :w] = meta["block_tables"][:, :w]
        h["context_lens"][:B] = meta["context_lens"]; h["context_lens"][B:] = 0
        h["query_start_loc"][: B + 1] = meta["query_start_loc"]; h["query_start_loc"][B + 1:] = T
        h["seq_order"][:] = np.argsort(-h["context_lens"], kind="stable")  # longest context first
        return self._commit(T, B, input_ids)

    def load_requests(self, requests: Sequence[dict], input_ids: np.ndarray, page_size: int) -> tuple[int, int, int]:
        """Build the step's metadata with the bucket padding straight into the staging buffer
        (native, one pass) and copy it to the device. Returns (tokens, sequences, max_seqlen_q)."""
        p = self._host_ptr
        T, maxq = _native_step_metadata(requests, page_size, self.max_blocks, self.num_tokens, self.num_seqs,
                                        p["positions"], p["slot_mapping"], p["query_start_loc"], p["context_lens"],
                                        p["block_tables"], p["seq_order"])
        if len(input_ids) != T:
            raise ValueError(f"{len(input_ids)} input ids for a step of {T} tokens")
        self._commit(T, len(requests), input_ids)
        return T, len(requests), maxq

    def _commit(self, T: int, B: int, input_ids) -> tuple[int, int]:
        ids = self._host["input_ids"]
        ids[:T] = input_ids
        ids[T:] = 0
        self.meta_dev.copy_(self.meta_host, non_blocking=False)
        return T, B


class Qwen3MoeDecoder:
    """Owns weights, the paged KV cache and per-bucket buffers / graphs."""

    def __init__(self, cfg: DecoderConfig, weights: DecoderWeights, num_cache_blocks: int, device="cuda"):
        self.cfg, self.w, self.device = cfg, weights, device
        self.cos, self.sin = rope_tables(cfg, device)
        # Physically [blocks, Hkv, 2, page, D]: one kv head's 16-key page of K and of V are two adjacent 4 KB pieces of
        # contiguous HBM for the wavefront that reads them (head-major alone: 8 % faster decode attention than
        # token-major; K and V adjacent: another ~1 %). The kernels see the usual [blocks, page, Hkv, D] views.
        shape = (num_cache_blocks, cfg.num_kv_heads, 2, cfg.page_size, cfg.head_dim)
        self._kv = [torch.zeros(shape, dtype=torch.bfloat16, device=device) for _ in range(cfg.num_layers)]
        self.key_cache = [t[:, :, 0].permute(0, 2, 1, 3) for t in self._kv]
        self.value_cache = [t[:, :, 1].permute(0, 2, 1, 3) for t in self._kv]
        self.buffers: dict[tuple[int, int], StepBuffers] = {}
        self.graphs: dict[tuple, torch.cuda.CUDAGraph] = {}
        self.prefetch_next_qkv = True  # see forward(): a cache hint, never a result
        self._attn_ws: Optional[torch.Tensor] = None

    def bucket(self, num_tokens: int, num_seqs: int) -> StepBuffers:
        key = (num_tokens, num_seqs)
        if key not in self.buffers:
            b = self.buffers[key] = StepBuffers(self.cfg, num_tokens, num_seqs, self.device,
                                                packed_only=self.w.packed_only, packed=self.w.packed is not None)
            # Steps run one at a time on one stream, so buckets share one decode-attention workspace. A bucket
            # that needs more than the shared one holds gets a new, larger one, which later buckets share;
            # earlier buckets (and graphs captured on them) keep the tensor they were given.
            if b.attn_ws_bytes > 0:
                if self._attn_ws is None or self._attn_ws.numel() < b.attn_ws_bytes:
                    self._attn_ws = torch.empty(b.attn_ws_bytes, dtype=torch.uint8, device=self.device)
                b.attn_ws = self._attn_ws
        return self.buffers[key]

    # ---- one forward pass over a bucket's static buffers (capture-safe: no sync, no host reads)
    def forward(self, b: StepBuffers, max_seqlen_q: int, routing_log: Optional[list] = None) -> None:
        cfg, w = self.cfg, self.w
        scale = cfg.head_dim ** -0.5
        E, k, I = cfg.num_experts, cfg.top_k, cfg.moe_intermediate
        ops.embedding(w.embed, b.input_ids, out=b.x)
        for li, lw in enumerate(w.layers):
            if li == 0:
                ops.rms_norm(b.x, lw["in_norm"], cfg.rms_eps, hf_two_rounding=True, out=b.h)
            ops.gemm_nt(b.h, lw["qkv"], out=b.qkv)
            ops.qk_norm_rope_store(b.qkv, lw["q_norm"], lw["k_norm"], self.cos, self.sin, b.positions, b.slot_mapping,
                                   b.q, self.key_cache[li], self.value_cache[li], cfg.num_heads, cfg.num_kv_heads,
                                   cfg.head_dim, cfg.rms_eps)
            ops.paged_attention(b.q, self.key_cache[li], self.value_cache[li], b.query_start_loc, b.context_lens,
                                b.block_tables, scale, max_seqlen_q, out=b.attn, workspace=b.attn_ws,
                                seq_order=b.seq_order if max_seqlen_q == 1 else None)
            ops.gemm_nt(b.attn.view(b.num_tokens, -1), lw["o"], out=b.o)
            # x <- x + o ; h <- post_norm(x)
            ops.rms_norm(b.o, lw["post_norm"], cfg.rms_eps, hf_two_rounding=True, residual=b.x, sum_out=b.x, out=b.h)
            ops.gemm_nt(b.h, lw["router"], out=b.router_logits)
            self._router(b)
            if routing_log is not None:  # debugging / tests only (allocates; not for graph capture)
                routing_log.append(b.topk_idx.clone())
            r = ops.moe_route(b.topk_idx, E, bm=b.bm, buffers=b.route_ints)
            if w.packed is not None and (r.bm <= 64 or r.bm == 256):
                pgu, pdn = w.packed[li]
                ops.moe_gemm_packed(b.h, pgu.rows(0, I), r, w2=pgu.rows(I, 2 * I), row_src=r.sorted_token,
                                    row_scale=b.topk_w, row_scale_idx=r.sorted_flat, out=b.hw)
                ops.moe_gemm_packed(b.hw, pdn, r, out=b.eo)
            else:
                gu = lw["gate_up"]
                if gu is None:
                    raise RuntimeError(f"bucket with {r.bm}-row expert tiles was made before the [E, N, K] expert "
                                       "tensors were freed: make buckets after pack_experts(keep_unpacked=False)")
                ops.moe_gemm(b.h, gu[:, :I, :], r, w2=gu[:, I:, :], row_src=r.sorted_token, row_scale=b.topk_w,
                             row_scale_idx=r.sorted_flat, out=b.hw)
                ops.moe_gemm(b.hw, lw["down"], r, out=b.eo)
            nxt = w.layers[li + 1]["in_norm"] if li + 1 < cfg.num_layers else w.final_norm
            # x <- x + sum_slots(eo) ; h <- next norm(x)
            # decode-sized steps read the next layer's qkv weights cold: spare workgroups of the combine fetch them
            pf = w.layers[li + 1]["qkv"] if (self.prefetch_next_qkv and li + 1 < cfg.num_layers and b.num_tokens <= 512) else None
            ops.moe_gather(b.eo, r.scatter_index, residual=b.x, out=b.x, norm_weight=nxt, norm_out=b.h,
                           eps=cfg.rms_eps, hf_two_rounding=True, prefetch=pf)

    def _router(self, b: StepBuffers) -> None:
        from . import _lib

        cfg = self.cfg
        _lib.check(
            _lib.load().vx_router_topk(
                b.router_logits.data_ptr(), b.topk_w.data_ptr(), b.topk_idx.data_ptr(), b.num_tokens, cfg.num_experts,
                cfg.top_k, b.router_logits.stride(0), 1, 1, 0, int(cfg.norm_topk_prob),
                torch.cuda.current_stream().cuda_stream),
            "vx_router_topk",
        )

    def sample(self, b: StepBuffers, decode: bool, sampling: Optional[tuple] = None) -> None:
        """Last token of each sequence -> lm_head -> token and its fp32 logprob. ``sampling`` is
        ``None`` for greedy decoding or ``(temperature, top_k, top_p)``: then row s draws its token
        with the noise stream of (``b.seeds[s]``, its context length), whatever batch it is in."""
        if decode and b.num_tokens == b.num_seqs:
            last = b.h  # every token is a last token
        else:
            idx = (b.query_start_loc[1:].long() - 1).clamp_(min=0)
            torch.index_select(b.h, 0, idx, out=b.last_h)
            last = b.last_h
        ops.gemm_nt(last, self.w.lm_head, out=b.logits)
        if sampling is None:
            lp, tok = ops.logprobs(b.logits, None, return_tokens=True)
            b.tokens.copy_(tok)
        else:
            temperature, top_k, top_p = sampling
            b.sample_pos.copy_(b.context_lens)
            ops.sample_tokens(b.logits, temperature, top_k, top_p, b.seeds, b.sample_pos, out=b.tokens)
            lp = ops.logprobs(b.logits, b.tokens)
        b.logprobs.copy_(lp)

    def step(self, b: StepBuffers, max_seqlen_q: int, routing_log: Optional[list] = None,
             sampling: Optional[tuple] = None) -> None:
        self.forward(b, max_seqlen_q, routing_log)
        self.sample(b, decode=(max_seqlen_q == 1), sampling=sampling)

    def capture(self, b: StepBuffers, max_seqlen_q: int = 1, sampling: Optional[tuple] = None) -> torch.cuda.CUDAGraph:
        key = (b.num_tokens, b.num_seqs, max_seqlen_q, sampling)
        if key in self.graphs:
            return self.graphs[key]
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            self.step(b, max_seqlen_q, sampling=sampling)  # warm-up on a side stream
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self.step(b, max_seqlen_q, sampling=sampling)
        self.graphs[key] = g
        return g


def decode_bytes_per_step(cfg: DecoderConfig, context_lens: Sequence[int], experts_hit_per_layer: Optional[int] = None) -> dict:
    """Algorithmic HBM bytes of one decode step: every weight touched once plus the KV of every
    sequence, plus small activation terms."""
    H, D, E, I, V = cfg.hidden_size, cfg.head_dim, cfg.num_experts, cfg.moe_intermediate, cfg.vocab_size
    B = len(context_lens)
    U = E if experts_hit_per_layer is None else experts_hit_per_layer
    attn_w = (cfg.qkv_dim * H + H * cfg.num_heads * D) * 2
    router_w = E * H * 2
    expert_w = U * 3 * H * I * 2
    kv = int(sum(context_lens)) * 2 * cfg.num_kv_heads * D * 2
    per_layer = attn_w + router_w + expert_w + kv
    head = V * H * 2 + B * V * 2
    return {"weights": cfg.num_layers * (attn_w + router_w + expert_w) + V * H * 2, "kv": cfg.num_layers * kv,
            "total": cfg.num_layers * per_layer + head, "moe_per_layer": expert_w, "kv_per_layer": kv}
