/*
 * vexact_hip.h - C ABI of libvexact_hip.so: hand-written gfx950 (MI355X) kernels for the
 * batch-invariant inference hot path of verl-project/vexact.
 *
 * Conventions (every entry point):
 *   - returns 0 on success or a negative VX_ERR_* code; never throws, never allocates, never
 *     synchronises and never reads device memory on the host, so every call is safe under HIP
 *     graph capture;
 *   - all data pointers are device pointers owned by the caller; `stream` is the HIP stream to
 *     launch on; strides and leading dimensions are in ELEMENTS unless the name says bytes;
 *   - launch geometry depends only on the sizes passed by value, never on device data;
 *   - dtype codes: 0 = float32, 1 = bfloat16, 2 = float16, except where an entry point states its own (the typed
 *     attention entry points, which grew out of a bf16-only form: 0 = bfloat16, 1 = float16, 2 = float32);
 *   - batch invariance: the bits of an output row depend on that row's own inputs only (not on
 *     the number of rows, their order, or which other rows share the launch).
 *
 * The reference has no C FFI; each entry point names the Python/Triton function of
 * /root/reference it replaces (file:line).
 */
#ifndef VEXACT_HIP_H_
#define VEXACT_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* hipStream_t;

#define VX_OK 0
#define VX_ERR_ARG (-1)         /* null pointer, negative size, bad stride */
#define VX_ERR_UNSUPPORTED (-2) /* shape / dtype / alignment / layout outside the fast paths */
#define VX_ERR_WORKSPACE (-3)   /* workspace pointer missing or too small */
#define VX_ERR_LAUNCH (-4)      /* hipLaunch reported an error */

int vx_abi_version(void);
const char* vx_status_string(int code);

/* ---- row reductions ------------------------------------------------------------------- */

/* mean over the middle dim of an (M, N, K) strided view, output (M, K) with strides (o0, o1).
 * Replaces mean_kernel / mean_dim, vexact/batch_invariant_ops/batch_invariant_ops.py:336-473. */
int vx_mean_dim(const void* in, void* out, int dtype, int64_t M, int64_t N, int64_t K, int64_t s0,
                int64_t s1, int64_t s2, int64_t o0, int64_t o1, hipStream_t stream);

/* RMSNorm over the last dim of [rows, n].
 *   mode 0: y = round(x * (1/sqrt(mean(x^2) + eps)) * w)          (one rounding)
 *           replaces _rms_norm_kernel / _rms_norm_forward, batch_invariant_ops.py:637-687
 *   mode 1: y = round(w * round(x * rsqrt(mean(x^2) + eps)))      (HuggingFace Qwen3 RMSNorm as it
 *           executes when its .mean(-1) is routed through mean_dim, batch_invariant_ops.py:619-622;
 *           rsqrt = the double-precision quotient 1/sqrt rounded once to fp32, which is what
 *           torch.rsqrt returns on this GPU, so the result has the bits of the module's forward)
 * residual (optional): the row is first replaced by round(x + residual) and that sum is written to
 * sum_out (optional; may alias x or residual). */
int vx_rms_norm(const void* x, const void* residual, const void* weight, void* y, void* sum_out,
                int dtype, int64_t rows, int64_t n, int64_t x_stride, int64_t res_stride,
                int64_t y_stride, int64_t sum_stride, float eps, int mode, hipStream_t stream);

/* log_softmax over the last dim of [rows, n]; needs vx_log_softmax_workspace_bytes(rows, n) bytes.
 * Replaces _log_softmax_kernel / log_softmax, batch_invariant_ops.py:231-333. */
int64_t vx_log_softmax_workspace_bytes(int64_t rows, int64_t n);
int vx_log_softmax(const void* x, void* y, int dtype, int64_t rows, int64_t n, int64_t x_stride,
                   int64_t y_stride, void* workspace, int64_t workspace_bytes, hipStream_t stream);

/* out[i] = logits[i, labels[i]] - logsumexp(logits[i, :]) in fp32 (same workspace as log_softmax).
 * labels == NULL: use the first argmax of the row (greedy token), also written to tokens_out.
 * Replaces logprobs_from_logits_flash_attn, vexact/batch_invariant_ops/standalone_logprobs.py:28-55. */
int vx_logprobs(const void* logits, const int64_t* labels, float* out, int64_t* tokens_out, int dtype,
                int64_t rows, int64_t n, int64_t x_stride, void* workspace, int64_t workspace_bytes,
                hipStream_t stream);

/* Backward of vx_rms_norm without residual (the training side of batch_invariant_rms_norm / of the HuggingFace
 * RMSNorm forward that mode 1 restates), bf16 or fp16, n % 8 == 0, n <= 8192: d_x = inv (d_h - h mean(d_h h)) with
 * h = x inv, d_h = d_y w; d_w = sum over rows of d_y r(h) (mode 1) or d_y h (mode 0), accumulated in fp32 in a fixed
 * order (deterministic for a given number of rows). Workspace: vx_rms_norm_bwd_workspace_bytes(rows, n). */
int64_t vx_rms_norm_bwd_workspace_bytes(int64_t rows, int64_t n);
int vx_rms_norm_bwd(const void* x, const void* weight, const void* dy, void* dx, void* dw, int dtype, int64_t rows,
                    int64_t n, int64_t x_stride, int64_t dy_stride, int64_t dx_stride, float eps, int mode,
                    void* workspace, int64_t workspace_bytes, hipStream_t stream);

/* Gradient of vx_logprobs with respect to the logits (the backward of the cross-entropy kernel behind the
 * reference's logprobs_from_logits_flash_attn, standalone_logprobs.py:28-55, whose inplace_backward writes it into the
 * logits): d_logits[i, j] = d_out[i] ((j == labels[i]) - softmax(logits[i])[j]), from the forward's out (which fixes
 * logsumexp). d_logits may be logits itself. At most 65535 rows per call. */
int vx_logprobs_bwd(const void* logits, const int64_t* labels, const float* out, const float* d_out, void* d_logits,
                    int dtype, int64_t rows, int64_t n, int64_t x_stride, int64_t d_stride, hipStream_t stream);

/* vx_logprobs for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc): no workspace argument, no counterpart in the reference. The chunk partials live in a
 * 1 MiB array inside the library's device image (VX_LOGPROBS_STATIC_BYTES; every GPU the library runs on holds
 * it until the process ends), so rows * ceil(n / 4096) * 16 bytes must not exceed that: 256 rows of a
 * 151936-entry vocabulary need 152 KiB. Larger problems return VX_ERR_WORKSPACE before anything is launched.
 * Calls no hipMalloc / hipFree or other allocating routine; the first call on a device looks the array's address
 * up once (make that call outside a capture). Same kernels and same bits as vx_logprobs. All calls on one GPU
 * share the array: calls that overlap on one GPU (different streams, different threads) race; calls on one
 * stream are ordered and safe. Nothing in the array has to be cleared between calls. */
#define VX_LOGPROBS_STATIC_BYTES (1 << 20)
int vx_logprobs_static(const void* logits, const int64_t* labels, float* out, int64_t* tokens_out, int dtype,
                       int64_t rows, int64_t n, int64_t x_stride, hipStream_t stream);

/* ---- dense GEMM ----------------------------------------------------------------------- */

/* C[M,N] = X[M,K] * W[N,K]^T (+ bias[N]), bf16 in/out, fp32 accumulate, K ascending, no split-K.
 * Needs K % 8 == 0, ldx % 8 == 0, ldw % 8 == 0 and 16-byte aligned X, W (else VX_ERR_UNSUPPORTED).
 * Replaces matmul_kernel_persistent / matmul_persistent, batch_invariant_ops.py:53-228. */
int vx_gemm_bf16_nt(const void* x, const void* w, const void* bias, void* c, int64_t M, int64_t N,
                    int64_t K, int64_t ldx, int64_t ldw, int64_t ldc, hipStream_t stream);
/* Same, forcing the kernel: kind 0 = weight-streaming with 16*mt-row tiles (mt in 1,2,4),
 * kind 1 = 128x128 LDS-tiled, kind 2 = weight-streaming with 16 k-steps in flight, kind 3 = 256x256
 * persistent tiles with direct-to-LDS loads (needs K % 64 == 0 and operands below 4 GiB, else
 * VX_ERR_UNSUPPORTED), kind 4 = LDS ring kernel for 65..512 rows, mt = configuration 0..6 (K % 64,
 * 128 or 256 == 0 depending on the configuration). Results are bit-identical across kinds (tested). */
int vx_gemm_bf16_nt_variant(const void* x, const void* w, const void* bias, void* c, int64_t M,
                            int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldc, int kind,
                            int mt, hipStream_t stream);
/* Dense SwiGLU: C[M, N] = r16(r16(silu(r16(X Wg^T))) * r16(X Wu^T)) for K-contiguous bf16 X [M, K],
 * Wg, Wu [N, K] (same pitch ldw): gate_proj, up_proj and act_fn(gate) * up of a dense MLP in one
 * kernel, bit-identical to two vx_gemm_bf16_nt calls followed by bf16 silu and multiply (the glue
 * the reference runs in torch between its GEMMs: Qwen3MoeMLP.forward, HF modeling_qwen3_moe.py, which
 * vexact/models/qwen3_moe/modeling_qwen3_moe.py keeps for the dense layers). kind < 0 chooses the
 * kernel by M; 0 (with mt = 1 / 2 / 4: 16 mt rows per tile), 1, 3 force the streaming, 128x128 tiled
 * or 256x256 wide kernel (all give the same bits). */
int vx_gemm_swiglu_bf16_nt(const void* x, const void* w_gate, const void* w_up, void* c, int64_t M, int64_t N,
                           int64_t K, int64_t ldx, int64_t ldw, int64_t ldc, int kind, int mt, hipStream_t stream);

/* Batched, fully strided fallback for any dtype code: one thread per output, fp32 FMA chain in
 * ascending k. Covers the layouts / dtypes of matmul_persistent and _bmm_kernel / triton_bmm
 * (batch_invariant_ops.py:484-606) that the fast path rejects. */
int vx_gemm_generic(const void* a, const void* b, const void* bias, void* c, int dtype, int64_t batch,
                    int64_t M, int64_t N, int64_t K, int64_t sab, int64_t sam, int64_t sak,
                    int64_t sbb, int64_t sbk, int64_t sbn, int64_t scb, int64_t scm, int64_t scn,
                    hipStream_t stream);
/* C[M,N] = X[M,K] * W[N,K]^T (+ bias[N]) for float32 (dtype 0; true fp32 products, v_mfma_f32_16x16x4_f32) and
 * float16 (dtype 2; v_mfma_f32_16x16x32_f16): fp32 accumulate, K ascending, no split-K, one kernel and one tile
 * shape for every M, so a row's bits do not depend on the other rows. Strides in elements, K contiguous.
 * Replaces the fp16 / fp32 configurations of matmul_persistent, batch_invariant_ops.py:158-228 (tile table
 * :182-206; the reference's fp32 tl.dot default is TF32 on its hardware, not copied). */
int vx_gemm_nt_mfma(const void* x, const void* w, const void* bias, void* c, int dtype, int64_t M, int64_t N, int64_t K,
                    int64_t ldx, int64_t ldw, int64_t ldc, hipStream_t stream);
/* out[n, k] = in[k, n] (bf16) - packs a [K, N] row-major operand for vx_gemm_bf16_nt. */
int vx_transpose_bf16(const void* in, void* out, int64_t K, int64_t N, int64_t ld_in, int64_t ld_out,
                      hipStream_t stream);

/* ---- paged KV cache + attention -------------------------------------------------------- */

/* cache.view(-1, row)[slot_mapping[t]] = src[t] for slot != -1; value / v_cache may be NULL.
 * Replaces _store_cache_kernel / store_kvcache, vexact/batch_invariant_ops/kv_cache_context.py:259-314. */
int vx_store_kvcache(const void* key, const void* value, void* k_cache, void* v_cache,
                     const int* slot_mapping, int64_t num_tokens, int64_t k_src_stride_bytes,
                     int64_t v_src_stride_bytes, int64_t k_row_bytes, int64_t v_row_bytes,
                     hipStream_t stream);

/* The same scatter into caches that are [blocks, page_size, heads, D] views with the given byte strides (block,
 * in-page row, head; a head's D elements contiguous), e.g. of head-major memory [blocks, heads, page_size, D], which
 * the decode kernels stream faster than the reference's layout. slot = block * page_size + row. */
int vx_store_kvcache_strided(const void* key, const void* value, void* k_cache, void* v_cache, const int* slot_mapping,
                             int64_t num_tokens, int heads, int64_t k_src_stride_bytes, int64_t v_src_stride_bytes,
                             int64_t k_head_bytes, int64_t v_head_bytes, int page_size, int64_t k_block_stride_bytes,
                             int64_t k_row_stride_bytes, int64_t k_head_stride_bytes, int64_t v_block_stride_bytes,
                             int64_t v_row_stride_bytes, int64_t v_head_stride_bytes, hipStream_t stream);

/* Causal GQA attention, bf16, head dims (Dk, Dv) in {(32,32),(64,64),(128,128),(192,128),(256,256)}.
 *   mode 0: paged decode - every sequence has at most one query token; KV is split into fixed
 *           256-key chunks (absolute positions) and folded in ascending order; needs
 *           vx_paged_attn_decode_workspace_bytes(num_seqs, Hq, Hkv, Dv, max_pages * page_size) bytes
 *           (modes 3 and 4 are mode 0 with the kernel forced: 3 = one wavefront per chunk plus a
 *           combine launch, 4 = chunks folded inside one workgroup per (sequence, kv head); mode 0
 *           takes 4 when num_seqs * Hkv fills the machine. The results are bit-identical.)
 *   mode 1: paged general (chunked prefill, mixed batches) - same arithmetic per row as mode 0. Sequences
 *           with exactly one query row (decode tokens beside prefill chunks; a whole decode batch that a
 *           captured graph launches with max_seqlen_q = its bucket's tokens) run on the mode-4 kernel
 *           inside the same call when that form fits and no lse is asked for; the other sequences' row
 *           blocks are numbered compactly when ceil(max_seqlen_q / rows per block) * num_seqs would mostly
 *           be empty workgroups. Neither changes a bit.
 *   mode 2: packed K/V [Tk, Hkv, D] with cu_seqlens_k (skp = row stride, no block table)
 * q [total_q, Hq, Dk], k/v cache [blocks, page, Hkv, D], out [total_q, Hq, Dv];
 * query i of a sequence sits at absolute position kv_len - q_len + i.
 * Replaces _paged_attn_fwd_block_kernel / _PagedFlashAttentionVarlen.forward and the forward of
 * _varlen_attn_fwd_block_kernel, vexact/batch_invariant_ops/triton_invariant_attention.py:433-692, 47-190. */
int vx_attn_chunk_size(void);
int64_t vx_paged_attn_decode_workspace_bytes(int64_t num_seqs, int64_t Hq, int64_t Hkv, int64_t Dv,
                                             int64_t max_kv_len);
/* What a launch with this mode really uses: 0 when it takes the fused form (mode 4, or mode 0 with
 * num_seqs * Hkv >= 256), whose chunk states stay in LDS; then workspace may be NULL. The _bytes figure
 * above is enough for every mode.
 * Rows of a sequence that has query tokens but no key at all (seqused_k <= 0) are left unwritten in every
 * mode, like the reference, whose grid has no block for them; query rows in front of the first key
 * (q_len > kv_len) are written as 0 by the general kernels. Padded sequences (q_len = 0) write nothing. */
int64_t vx_paged_attn_decode_workspace_needed(int64_t num_seqs, int64_t Hq, int64_t Hkv, int64_t Dv,
                                              int64_t max_kv_len, int mode);
int vx_attention(const void* q, const void* k, const void* v, void* out, const int* cu_seqlens_q,
                 const int* seqused_k, const int* cu_seqlens_k, const int* block_table,
                 int64_t total_q, int64_t num_seqs, int Hq, int Hkv, int Dk, int Dv, int64_t sqt,
                 int64_t sqh, int64_t skb, int64_t skp, int64_t skh, int64_t svb, int64_t svp,
                 int64_t svh, int64_t sot, int64_t soh, int64_t bt_stride, int64_t max_pages,
                 int page_size, float softmax_scale, int causal, int mode, int max_seqlen_q,
                 void* workspace, int64_t workspace_bytes, hipStream_t stream);

/* vx_attention with two optional extras.
 * lse [total_q, Hq] fp32 (modes 1 and 2): each query row's log-sum-exp (m + log2 l) ln 2, as the
 * reference's packed forward saves it (_varlen_attn_fwd_block_kernel,
 * triton_invariant_attention.py:187-191); +inf for a row without a visible key.
 * seq_order [num_seqs] int32 (paged modes 0, 1, 3, 4): a permutation of the sequences; workgroup i of
 * the decode kernels takes sequence seq_order[i] (in mode 1: of the decode kernel that takes the sequences
 * of one query row). Longest context first shortens the tail of a batch with mixed lengths; the results do
 * not depend on it. (No counterpart in the reference.) */
int vx_attention_ex(const void* q, const void* k, const void* v, void* out, float* lse, const int* seq_order,
                    const int* cu_seqlens_q, const int* seqused_k, const int* cu_seqlens_k, const int* block_table,
                    int64_t total_q, int64_t num_seqs, int Hq, int Hkv, int Dk, int Dv,
                    int64_t sqt, int64_t sqh, int64_t skb, int64_t skp, int64_t skh, int64_t svb,
                    int64_t svp, int64_t svh, int64_t sot, int64_t soh, int64_t bt_stride,
                    int64_t max_pages, int page_size, float softmax_scale, int causal, int mode,
                    int max_seqlen_q, void* workspace, int64_t workspace_bytes, hipStream_t stream);

/* vx_attention_ex for either 16-bit element type (dtype 0 = bf16, 1 = fp16; q, k, v and out share it) and any
 * head sizes Dk, Dv <= 256: the reference's kernels mask the head dimension to the next power of two and take
 * fp16 or bf16 (triton_invariant_attention.py:98-103, 485-490, 645-649). bf16 at (Dk, Dv) in {(32, 32), (64, 64),
 * (128, 128), (192, 128), (256, 256)} with 16-byte addressable rows runs kernels built for exactly those sizes
 * (this is what vx_attention / vx_attention_ex call); every other case runs the kernels built for the next of
 * (64, 64), (128, 128), (256, 128), (256, 256) with the missing query columns as zeros, which leaves every bit
 * as an exact-size kernel would compute it; head sizes or strides that are not multiples of 8 elements, or bases
 * that are not 16-byte aligned, are served with per-element accesses (correct, slow). dtype 2 = fp32, which the
 * reference's kernels also take (FP32_OUTPUT, triton_invariant_attention.py:108-113; its backward tests run in it):
 * a correctness path of one thread per output row, single ascending fp32 sums and true fp32 products (the
 * reference's tl.dot would use TF32), every mode through the same routine, so paged, packed, prefill and decode
 * agree bit for bit; it needs no workspace and ignores seq_order. Any other dtype code: VX_ERR_UNSUPPORTED. */
int vx_attention_typed(const void* q, const void* k, const void* v, void* out, float* lse, const int* seq_order,
                       const int* cu_seqlens_q, const int* seqused_k, const int* cu_seqlens_k, const int* block_table,
                       int64_t total_q, int64_t num_seqs, int Hq, int Hkv, int Dk, int Dv,
                       int64_t sqt, int64_t sqh, int64_t skb, int64_t skp, int64_t skh, int64_t svb,
                       int64_t svp, int64_t svh, int64_t sot, int64_t soh, int64_t bt_stride,
                       int64_t max_pages, int page_size, float softmax_scale, int causal, int mode,
                       int max_seqlen_q, int dtype, void* workspace, int64_t workspace_bytes, hipStream_t stream);

/* Backward of causal varlen attention on packed q [Tq, Hq, D], k / v [Tk, Hkv, D] (bf16, D = 64 or 128):
 * dq, dk, dv (bf16) from dout, the forward's out and lse. P and dS are rounded to bf16 before they
 * enter a matrix product, as in the reference; all sums run in an order fixed by the sequence's own
 * lengths. strides[16] = token and head strides (elements) of q, k, v, out, dout, dq, dk, dv.
 * Workspace: vx_attention_bwd_workspace_bytes(total_q, Hq) (the row sums O . dO).
 * Replaces _varlen_attn_bwd_dq_kernel / _varlen_attn_bwd_dkv_kernel and
 * _NonpagedFlashAttentionVarlen.backward (triton_invariant_attention.py:193-430, 786-902). */
int64_t vx_attention_bwd_workspace_bytes(int64_t total_q, int64_t Hq);
int vx_attention_bwd(const void* q, const void* k, const void* v, const void* out, const void* dout, const float* lse,
                     void* dq, void* dk, void* dv, const int* cu_seqlens_q, const int* cu_seqlens_k,
                     int64_t total_q, int64_t total_k, int64_t num_seqs, int Hq, int Hkv, int D,
                     const int64_t* strides, float softmax_scale, int max_seqlen_q, int max_seqlen_k,
                     void* workspace, int64_t workspace_bytes, hipStream_t stream);
/* The same for either 16-bit element type (dtype 0 = bf16, 1 = fp16) and any head sizes up to 256: Dk of
 * q / k / dq / dk, Dv of v / out / dout / dv, as _NonpagedFlashAttentionVarlen.backward takes them
 * (triton_invariant_attention.py:786-902, BLOCK_D = next power of two of the larger one). bf16 at Dk = Dv = 128
 * runs the LDS kernels, everything else register-form kernels built for 64, 128 or 256 (the last two spill and
 * are slow); rows that are not 16-byte addressable are served per element. dtype 2 = fp32 (every tensor fp32):
 * one thread per gradient row, P recomputed from lse in fp32 without intermediate rounding. */
int vx_attention_bwd_typed(const void* q, const void* k, const void* v, const void* out, const void* dout, const float* lse,
                           void* dq, void* dk, void* dv, const int* cu_seqlens_q, const int* cu_seqlens_k,
                           int64_t total_q, int64_t total_k, int64_t num_seqs, int Hq, int Hkv, int Dk, int Dv,
                           const int64_t* strides, float softmax_scale, int max_seqlen_q, int max_seqlen_k, int dtype,
                           void* workspace, int64_t workspace_bytes, hipStream_t stream);

/* ---- fused MoE ------------------------------------------------------------------------- */

/* softmax(fp32) -> top-k (ties: lower expert first) -> optional renorm -> cast.
 * Replaces the router in moe_block_forward, vexact/models/qwen3_moe/modeling_qwen3_moe.py:128-134. */
int vx_router_topk(const void* logits, void* weights_out, void* idx_out, int64_t T, int E, int k,
                   int64_t ld, int logits_bf16, int out_bf16, int idx_i64, int renorm,
                   hipStream_t stream);

/* Routing integers for T*k flat entries (all exact): splits[E], cu[E+1], scatter_index[T*k] (stable
 * expert-major rank), sorted_token[T*k], sorted_flat[T*k], and a tile table of at most
 * vx_moe_max_tiles(T*k, E, bm) row tiles (group id or -1, first row, rows).
 * Replaces expert_histogram (group_gemm/kernel/moe.py:52-81), the double argsort
 * (fused_moe.py:43) and _build_moe_indices (fused_moe.py:268-292). */
int64_t vx_moe_max_tiles(int64_t n_entries, int E, int bm);
int vx_moe_route(const void* expert_idx, int idx_i64, int64_t T, int k, int E, int bm, int* splits,
                 int* cu, int* scatter_index, int* sorted_token, int* sorted_flat, int* tile_group,
                 int* tile_row0, int* tile_rows, int64_t max_tiles, hipStream_t stream);
/* The same with a workspace of vx_moe_route_workspace_bytes(T * k, E) bytes (0 below 3072 entries): from
 * 3072 entries on the work is spread over chunks of 1024 entries in three launches (per-chunk counts,
 * one scan, per-chunk stable ranks) instead of one workgroup; identical integers. */
int64_t vx_moe_route_workspace_bytes(int64_t n_entries, int E);
int vx_moe_route_ws(const void* expert_idx, int idx_i64, int64_t T, int k, int E, int bm, int* splits,
                    int* cu, int* scatter_index, int* sorted_token, int* sorted_flat, int* tile_group,
                    int* tile_row0, int* tile_rows, int64_t max_tiles, void* workspace, int64_t workspace_bytes,
                    hipStream_t stream);

/* Grouped GEMM over the tile table: C[rows] = X[row_src[rows]] * W[group]^T, bf16.
 *   epi 0: plain store (replaces group_gemm_same_nk, group_gemm/kernel/group_gemm.py:65-237)
 *   epi 1: w = gate rows, w2 = up rows, C = round(round(round(silu(round(g))) * round(u)) * s) with
 *          s = row_scale[row_scale_idx[row]] (adds the glue of fused_moe.py:75-88)
 * bm (rows per tile) must match the tile table: 16 / 32 / 64 stream weights, 128 is LDS-tiled,
 * 256 uses 256x256 tiles with direct-to-LDS loads (prefill sizes; needs K % 64 == 0 and x_rows = the
 * number of rows addressable in x, which bounds its 32-bit load offsets; other bm ignore x_rows). */
int vx_moe_gemm(const void* x, int64_t ldx, const void* w, const void* w2, int64_t ldw,
                int64_t w_gstride, void* c, int64_t ldc, int64_t N, int64_t K, const int* tile_group,
                const int* tile_row0, const int* tile_rows, int64_t max_tiles, int bm,
                const int* row_src, const void* row_scale, const int* row_scale_idx, int epi, int64_t x_rows,
                hipStream_t stream);

/* Fragment-order ("packed") copy of [G][N][K] bf16 weights for the weight-streaming kernels, made once per
 * weight update. No counterpart in the reference (its grouped GEMM, group_gemm/kernel/group_gemm.py:65-153,
 * reads [E, N, K] as stored): the values and every product are the same, only the order in HBM differs, so
 * that a wavefront reads one linear run per 16 weight rows instead of 16 pitched rows.
 *   out[g][nb][c][lane][8] = W_g[16 nb + lane % 16][32 c + 8 (lane / 16) .. + 8], zero past N and K,
 *   nb < ceil(N / 16), c < vx_packed_kchunks(K) (K rounded up to a multiple of 256, in 32-wide chunks):
 *   G * ceil(N / 16) * vx_packed_kchunks(K) * 512 elements. */
int vx_packed_kchunks(int64_t K);
int vx_pack_weights(const void* w, int64_t ldw, int64_t w_gstride, int64_t G, int64_t N, int64_t K, void* out,
                    hipStream_t stream);
/* vx_moe_gemm on packed weights, bm in {16, 32, 64} (decode sizes) or 256 (prefill sizes: K % 64 == 0 and
 * x_rows as for vx_moe_gemm, and for epi 1 w2 must lie behind w within 4 GiB, as the up rows of one packed
 * gate/up tensor do; x_rows is ignored otherwise), so that a model needs no [E, N, K] copy beside the packed one.
 * w (and w2 for epi 1) point at the packed image of the projection's first row, which must lie a multiple of
 * 16 rows into the packed tensor; w_gstride = elements between consecutive experts there. Same bits as
 * vx_moe_gemm. */
int vx_moe_gemm_packed(const void* x, int64_t ldx, const void* w, const void* w2, int64_t w_gstride, void* c,
                       int64_t ldc, int64_t N, int64_t K, const int* tile_group, const int* tile_row0,
                       const int* tile_rows, int64_t max_tiles, int bm, const int* row_src, const void* row_scale,
                       const int* row_scale_idx, int epi, int64_t x_rows, hipStream_t stream);

/* Grouped products of the fused-MoE backward (FusedMoeExpertFunction.backward, fused_moe.py:126-265), bf16
 * with fp32 accumulation, over the same tile table / expert offsets as the forward.
 *   vx_moe_gemm_nn: C[rows of expert e] = A[a_src[rows]] W_e (+ A2[rows] W2_e): the data gradient through a
 *     weight stored [K, N] (N contiguous; group stride w_gstride). a_src, a2 / w2 optional. bm <= 128, or
 *     bm == 256 (tiles of the forward's wide kernel; same bits): then K and K2 must be multiples of 64 and
 *     a_rows = rows addressable in a (a_src values, or the sorted rows, lie below it; it bounds the kernel's
 *     32-bit offsets; ignored for bm <= 128).
 *   vx_moe_gemm_tn: dW_e[N, K] = sum over sorted rows cu[e] <= r < cu[e+1] of dY[dy_src[r], :]^T X[x_src[r], :]:
 *     the weight gradient (zeros for an expert without rows). The row gathers are optional. dy_rows / x_rows =
 *     rows addressable in dy / x (at least 1 each; they decide whether the 256 x 256-tile kernel's 32-bit
 *     offsets reach every row; 0 = unknown, the 128 x 128-tile kernel runs; same bits either way).
 * N, K and row strides must be multiples of 8 elements. Each output element is one ascending MFMA chain
 * (no atomics, no split contraction): results are deterministic and independent of the other experts. */
int vx_moe_gemm_nn(const void* a, int64_t lda, const int* a_src, const void* w, int64_t ldw, int64_t w_gstride,
                   int64_t K, const void* a2, int64_t lda2, const void* w2, int64_t ldw2, int64_t w2_gstride,
                   int64_t K2, void* c, int64_t ldc, int64_t N, const int* tile_group, const int* tile_row0,
                   const int* tile_rows, int64_t max_tiles, int bm, int64_t a_rows, hipStream_t stream);
/* Gradient of vx_router_topk's weights with respect to the logits (the router of the reference's block is softmax ->
 * top-k -> renormalise -> cast as differentiable tensor operations, modeling_qwen3_moe.py:128-134): idx = the
 * selected experts [T, k] int64, d_weights [T, k] (bf16 or fp32), d_logits [T, E] in the logits' type. E <= 512,
 * k <= 64. */
int vx_router_topk_bwd(const void* logits, const int64_t* idx, const void* d_weights, void* d_logits, int64_t T, int E,
                       int k, int64_t ld, int64_t ld_out, int logits_bf16, int weights_bf16, int renorm,
                       hipStream_t stream);
/* The elementwise step of the same backward between the products (fused_moe.py:150-250: silu, its derivative, the
 * routing-weight gradient), one launch, bf16 with a rounding wherever one of the reference's tensor operations
 * rounds. For sorted row r, w = rw[flat[r]]: hw = silu(g) u w; d_rw[flat[r]] = sum_i (silu(g) u)(d_hw);
 * d_u = silu(g) (d_hw w); d_g = silu'(g) ((d_hw w) u). g, u, d_hw and the outputs hw, d_g, d_u: [rows, I] with
 * row strides (multiples of 8; d_g and d_u may be the halves of one [rows, 2 I] buffer); rw, d_rw: bf16 arrays
 * indexed by flat (every flat index occurs once). I % 8 == 0. */
int vx_moe_swiglu_bwd(const void* g, const void* u, const void* d_hw, int64_t ldg, int64_t ldu, int64_t ldd,
                      const void* rw, const int* flat, void* hw, void* d_g, void* d_u, void* d_rw, int64_t ld_hw,
                      int64_t ld_dg, int64_t ld_du, int64_t rows, int64_t I, hipStream_t stream);
int vx_moe_gemm_tn(const void* dy, int64_t lddy, const int* dy_src, const void* x, int64_t ldx, const int* x_src,
                   void* dw, int64_t lddw, int64_t dw_gstride, int64_t N, int64_t K, const int* cu,
                   int64_t num_experts, int64_t dy_rows, int64_t x_rows, hipStream_t stream);

/* Replace expert_histogram / moe_scatter / moe_gather, group_gemm/kernel/moe.py:52-81, 304-335, 131-161.
 * vx_moe_gather: y[t] = round(sum_i x[index[t, i]]) in slot order (fp32); with residual:
 * y[t] = round(residual[t] + round(sum)). */
int vx_expert_histogram(const void* idx, int idx_i64, int64_t n, int E, int* out, hipStream_t stream);
int vx_moe_scatter(const void* x, void* out, const int* index, int64_t T, int k, int64_t H, int64_t ldx,
                   int64_t ldo, hipStream_t stream);
int vx_moe_gather(const void* x, const int* index, const void* residual, void* y, int64_t T, int k,
                  int64_t H, int64_t ldx, int64_t ldr, int64_t ldy, hipStream_t stream);
/* Same, and additionally h = RMSNorm(y) with norm_weight (mode as vx_rms_norm): the RMSNorm that
 * follows the MoE block in the decoder layer, fused; bit-identical to vx_moe_gather + vx_rms_norm. */
int vx_moe_gather_norm(const void* x, const int* index, const void* residual, void* y, int64_t T, int k,
                       int64_t H, int64_t ldx, int64_t ldr, int64_t ldy, const void* norm_weight, void* h,
                       int64_t ldh, float eps, int mode, hipStream_t stream);

/* vx_moe_gather_norm with a cache prefetch riding along: extra workgroups read `prefetch_bytes` (rounded down
 * to 16) from `prefetch` (16-byte aligned, readable) and discard them while the combine runs and leaves HBM
 * idle - e.g. the weights of the projection that follows, which it would otherwise read cold. Changes no
 * result; ignored on layouts the vector kernel cannot take. No counterpart in the reference. */
int vx_moe_gather_norm_prefetch(const void* x, const int* index, const void* residual, void* y, int64_t T, int k,
                                int64_t H, int64_t ldx, int64_t ldr, int64_t ldy, const void* norm_weight, void* h,
                                int64_t ldh, float eps, int mode, const void* prefetch, int64_t prefetch_bytes,
                                hipStream_t stream);

/* ---- decoder-layer glue ---------------------------------------------------------------- */

/* Per-head RMSNorm (mode 1 form) of q and k, bf16 rotary embedding from cos/sin tables
 * [max_pos, D], q -> q_out [T, Hq, D], k -> k_out (optional) and k_cache slot, v -> v_cache slot.
 * Both caches are [blocks, page_size, Hkv, D] views with the given element strides (block, in-page
 * row, head; D contiguous), so a head-major physical layout [blocks, Hkv, page_size, D] can be used.
 * qkv rows are [q heads | k heads | v heads]. positions may be null: row t of the tables is then token t's
 * (per-token cos / sin rows as HuggingFace's rotary module returns them). The scatter is store_kvcache
 * (kv_cache_context.py:294-314); norm + rotary are the HuggingFace Qwen3 attention prologue the
 * reference runs between its q/k/v projections and its attention call. */
int vx_qk_norm_rope_store(const void* qkv, int64_t ld, const void* q_norm_w, const void* k_norm_w,
                          const void* cos_table, const void* sin_table, const void* positions,
                          int pos_i64, const int* slot_mapping, void* q_out, void* k_out,
                          void* k_cache, void* v_cache, int64_t T, int Hq, int Hkv, int D, float eps,
                          int64_t max_pos, int page_size, int64_t cache_block_stride,
                          int64_t cache_row_stride, int64_t cache_head_stride, hipStream_t stream);
/* Rotary embedding alone, bf16: out[t, h, :] = r16(r16(x cos[t]) + r16(rotate_half(x) sin[t])) for x [T, H, D]
 * with element strides (token, head; D contiguous, D % 8 == 0) and per-token rows cos / sin [T, D] (row stride
 * cos_row_stride). One launch for what HuggingFace's apply_rotary_pos_emb (transformers modeling_qwen3_moe.py,
 * called between q/k norm and the attention function that the reference registers) does in five per tensor;
 * the reference's optional Liger patch swaps the same function (vexact/models/register.py:77-80). Same bits. */
int vx_rope(const void* x, void* out, const void* cos_rows, const void* sin_rows, int64_t T, int H, int D,
            int64_t x_token_stride, int64_t x_head_stride, int64_t out_token_stride, int64_t out_head_stride,
            int64_t cos_row_stride, hipStream_t stream);
int vx_embedding(const void* table, const void* ids, int ids_i64, void* out, int64_t T, int64_t H,
                 int64_t vocab, hipStream_t stream);
int vx_fill_i32(int* p, int value, int64_t n, hipStream_t stream);

/* ---- token sampler ------------------------------------------------------------------------- */

/* One token per row of logits [rows, V] (dtype 0 bf16, 1 fp32; ld = row pitch in elements):
 * x = f32(logit) * (1 / temperature); top_k (<= 0 or >= V: off) masks keys below the k-th largest;
 * top_p (>= 1: off) masks the keys whose inclusive ascending probability mass is <= 1 - p (integer
 * masses floor(exp(x - max) * 2^32), equal logits treated alike); the token is the winner of an
 * exponential race argmin E_i / exp(x_i - max) whose noise is Philox4x32-10 keyed by seeds[row] with
 * counter (token / 4, positions[row]), so it depends on (logits row, seed, position) only: not on
 * the batch or the row's place in it. Needs temperature > 0 and top_p > 0 (greedy decoding is
 * vx_logprobs with labels == NULL). No workspace, no host synchronisation.
 * Replaces Sampler.batch_sample_token / apply_top_k_top_p / _random_sample / _seeded_sample,
 * vexact/inferencer/sampler.py:29-189 (the seeded path there calls vLLM's Gumbel kernel). */
int vx_sample_tokens(const void* logits, int dtype, int64_t ld, int64_t rows, int64_t V, float temperature,
                     int top_k, float top_p, const int64_t* seeds, const int64_t* positions,
                     int64_t* tokens_out, hipStream_t stream);

/* ---- host-side step metadata and block allocator (CPU code, no device work, no stream) -------- */

/* Integer metadata of one step, written into host buffers sized for a graph bucket (cap_tokens
 * tokens, cap_seqs sequences): positions [cap_tokens] (int64), slot_mapping [cap_tokens],
 * query_start_loc [cap_seqs + 1], context_lens [cap_seqs], block_tables [cap_seqs, max_blocks].
 * Request s has context length num_computed[s] AFTER this step, tokens_this_step[s] query tokens
 * and the block ids block_ids[block_offsets[s] .. block_offsets[s + 1]). Padding: tokens past the
 * step get slot -1 / position 0; sequences past it get query_start_loc = total tokens, context
 * length 0 and an all-zero block-table row; unused entries of real rows are -1. seq_order [cap_seqs]
 * (optional) receives the sequences by context length, longest first (ties and padding in index
 * order), for vx_attention_ex.
 * Replaces _prepare_gen_ctx (vexact/inferencer/inferencer.py:193-291) and the static-buffer padding
 * of prepare_cudagraph_gen_ctx (inferencer.py:306-324) in one pass. VX_ERR_ARG if the step does not
 * fit the bucket or a request's blocks do not cover its context. */
int vx_host_step_metadata(int64_t num_reqs, const int64_t* num_computed, const int64_t* tokens_this_step,
                          const int32_t* block_ids, const int64_t* block_offsets, int32_t page_size,
                          int64_t max_blocks, int64_t cap_tokens, int64_t cap_seqs, int64_t* positions,
                          int32_t* slot_mapping, int32_t* query_start_loc, int32_t* context_lens,
                          int32_t* block_tables, int32_t* seq_order, int64_t* total_tokens, int32_t* max_seqlen_q);

/* Block allocator that always hands out the lowest free ids (KVCacheManager,
 * vexact/batch_invariant_ops/kv_cache_context.py:141-217). allocate: the blocks a request holding
 * num_current_blocks needs to cover total_tokens, ascending, into out; returns their number, 0 if
 * none are needed, -1 (nothing allocated) if too few are free or out_capacity is too small.
 * free: ids out of range or already free are ignored; returns the number freed. Not thread-safe. */
void* vx_kv_allocator_create(int64_t num_blocks);
void vx_kv_allocator_destroy(void* allocator);
int64_t vx_kv_allocator_num_free(const void* allocator);
int64_t vx_kv_allocator_allocate(void* allocator, int64_t total_tokens, int64_t num_current_blocks,
                                 int32_t page_size, int32_t* out, int64_t out_capacity);
int64_t vx_kv_allocator_free(void* allocator, const int32_t* ids, int64_t n);

#ifdef __cplusplus
}
#endif
#endif /* VEXACT_HIP_H_ */
