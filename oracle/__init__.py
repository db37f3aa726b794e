"""CPU oracle for the batch-invariant hot path: TEST INFRASTRUCTURE ONLY.

Plain torch-CPU / numpy restatements of the reference's algorithms (each function cites the
reference file:line it follows). Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this package; the product (``vexact_amd``) never
does, and has no CPU fallback.

How each function is pinned (checked in ``tests/test_oracle_*.py``; none needs the reference
imported, and the reference ships no stored golden vectors for these ops):

=====================  ===========================================================================
function               pinned by
=====================  ===========================================================================
matmul_ref             fp64 brute force on tiny inputs; exact integer-valued cases
mean_dim_ref           fp64 brute force; constant rows
rms_norm_ref (both)    fp64 brute force; unit-weight / constant-row closed forms; the two rounding
                       variants differ by <= 1 bf16 ulp
log_softmax_ref        torch.log_softmax (library routine); rows sum to 1 after exp; shift invariance
logprobs_ref           gather of log_softmax_ref; fallback formula the reference itself states
                       (standalone_logprobs.py:45-47)
store_kvcache_ref      python-loop restatement vs vectorised indexing; slot -1 rows untouched
paged gather           make_paged_kv_cache round trip (gather back == original sequences)
eager_attention        fp64 softmax-attention brute force; q_len = kv_len = 1 => out == v; uniform
                       keys => mean of visible values
router_ref             brute-force python top-k with the documented tie rule; weights sum to 1
routing_integers_ref   brute-force counting; numpy stable argsort twice (fused_moe.py:43)
fused_moe_ref          k=1,w=1 => plain SwiGLU MLP; all tokens on one expert => dense formula;
                       fp64 brute force on tiny shapes; HF-eager form within bf16 tolerance
prepare_gen_ctx_ref    hand-worked example; vectorised numpy twin
pad_for_graph_ref      hand-worked example (3 requests in a bucket of 8 tokens / 5 sequences) from the reference's
                       statements (inferencer.py:306-324), tests/test_host_logic.py
BlockAllocatorRef      hand-worked sequence on the restatement itself (lowest id first, out-of-blocks takes
                       nothing, double / foreign frees ignored), tests/test_host_logic.py
rope_tables_ref        HuggingFace Qwen3MoeRotaryEmbedding bit for bit (three theta / head sizes, positions to
                       40959); position 0 = identity, first pair turns by `position` radians
rope_ref               HuggingFace apply_rotary_pos_emb bit for bit; pair lengths preserved
qk_norm_rope_store_ref the HuggingFace attention module's own q_norm / k_norm (distinct non-unit weights) +
                       apply_rotary_pos_emb bit for bit; cache rows by slot, slot -1 and unmapped rows untouched
embedding_ref          torch indexing (library routine)
layer_ref              HuggingFace Qwen3MoeDecoderLayer on the CPU (eager attention, eager experts, norm weights in
                       [0.5, 1.5]): 0.8 % of the largest entry at worst (bound 2 %; swapped q/k norm weights: 4.3 %)
decoder_step_ref       HuggingFace Qwen3MoeForCausalLM last-token logits, packed prefill through the paged cache and
                       a decode step on top of it: logprob |d| <= 5e-2; a wrong rope_theta fails
attention_backward_ref autograd through the fp32 eager attention; one visible key => dV = dO, dQ = dK = 0
fused_moe_backward_ref autograd through an fp32 restatement of the expert MLPs
sampler.philox4x32     Random123 known-answer vectors
sampler.exp32 / log    numpy exp / log within 4e-7 / 2e-6; and, with the keys and Philox, bit for bit the text of the
                       kernel source's scalar routines compiled for the host (tests/test_oracle_sampler.py)
sampler.kept_mask_spec the reference's sort + cumsum rule (apply_top_k_top_p_ref) on tie-free rows
sample_tokens_ref      argmax(probs / q) with the same variates; softmax frequencies (chi-square
                       style bound); (seed, position) keyed: order invariance
=====================  ===========================================================================

Parity unpinned (arithmetic lives in third-party wheels that are not in the reference tree, and
only invariance tests cover them there): the exact bit patterns of flash-attn 3/4 attention,
flash-attn 2.8.4 cross-entropy, quack 0.3.4 grouped GEMM and veomni 0.1.9a5 fused MoE, and the noise stream of vLLM's seeded Gumbel sampling kernel. Parity
against those is by the closed forms above within the stated tolerances.
"""
