// Entry points of the attention kernels (attn_core.h) and the KV-cache row scatter. This file holds the bf16 kernels
// for the head sizes they are built for exactly; bf16 on other head sizes and fp16 live in paged_attn_pad.hip and
// paged_attn_f16.hip.
// Replaces _paged_attn_fwd_block_kernel / _PagedFlashAttentionVarlen
// (vexact/batch_invariant_ops/triton_invariant_attention.py:433-692), the forward of the packed
// twin _varlen_attn_fwd_block_kernel (:47-190, :700-784) and _store_cache_kernel / store_kvcache
// (vexact/batch_invariant_ops/kv_cache_context.py:259-314).
#include "attn_core.h"
#include "attn_f32_launch.h"

namespace vx {

// ---------------------------------------------------------------------------------------
// KV-cache scatter: cache.view(-1, row)[slot[t]] = src[t] for slot != -1. One wavefront per token
// copies row_bytes (multiple of 16) with 16-byte accesses.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void store_kv_kernel(const uint8_t* __restrict__ ksrc,
                                                       const uint8_t* __restrict__ vsrc,
                                                       uint8_t* __restrict__ kc, uint8_t* __restrict__ vc,
                                                       const int* __restrict__ slots, int64_t ntok,
                                                       int64_t ks_stride, int64_t vs_stride,
                                                       int k_row_bytes, int v_row_bytes) {
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= ntok) return;
  const int slot = slots[t];
  if (slot < 0) return;
  const int lane = threadIdx.x & 63;
  for (int b = lane * 16; b < k_row_bytes; b += 64 * 16)
    *(uint4*)(kc + (int64_t)slot * k_row_bytes + b) = *(const uint4*)(ksrc + t * ks_stride + b);
  if (vsrc)
    for (int b = lane * 16; b < v_row_bytes; b += 64 * 16)
      *(uint4*)(vc + (int64_t)slot * v_row_bytes + b) = *(const uint4*)(vsrc + t * vs_stride + b);
}

// The same scatter into a cache that is a [blocks, page, heads, D] view of other memory (head-major
// [blocks, heads, page, D], which decode attention streams faster): byte strides per block, in-page row and head.
// One wavefront per token; a lane moves 16 bytes of one head's row.
__global__ __launch_bounds__(256) void store_kv_strided_kernel(const uint8_t* __restrict__ ksrc,
                                                               const uint8_t* __restrict__ vsrc, uint8_t* __restrict__ kc,
                                                               uint8_t* __restrict__ vc, const int* __restrict__ slots,
                                                               int64_t ntok, int64_t ks_stride, int64_t vs_stride, int heads,
                                                               int k_head_bytes, int v_head_bytes, int page, int64_t kcb,
                                                               int64_t kcp, int64_t kch, int64_t vcb, int64_t vcp, int64_t vch) {
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= ntok) return;
  const int slot = slots[t];
  if (slot < 0) return;
  const int lane = threadIdx.x & 63;
  const int64_t blk = slot / page, row = slot % page;
  for (int b = lane * 16; b < heads * k_head_bytes; b += 64 * 16) {
    const int h = b / k_head_bytes, r = b - h * k_head_bytes;
    *(uint4*)(kc + blk * kcb + row * kcp + h * kch + r) = *(const uint4*)(ksrc + t * ks_stride + b);
  }
  if (vsrc)
    for (int b = lane * 16; b < heads * v_head_bytes; b += 64 * 16) {
      const int h = b / v_head_bytes, r = b - h * v_head_bytes;
      *(uint4*)(vc + blk * vcb + row * vcp + h * vch + r) = *(const uint4*)(vsrc + t * vs_stride + b);
    }
}

}  // namespace vx

using namespace vx;

extern "C" {

int vx_attn_chunk_size() { return ATT_CHUNK; }

int vx_attention_typed(const void* q, const void* k, const void* v, void* out, float* lse, const int* seq_order,
                       const int* cu_seqlens_q, const int* seqused_k, const int* cu_seqlens_k, const int* block_table,
                       int64_t total_q, int64_t num_seqs, int Hq, int Hkv, int Dk, int Dv,
                       int64_t sqt, int64_t sqh, int64_t skb, int64_t skp, int64_t skh, int64_t svb,
                       int64_t svp, int64_t svh, int64_t sot, int64_t soh, int64_t bt_stride,
                       int64_t max_pages, int page_size, float softmax_scale, int causal, int mode,
                       int max_seqlen_q, int dtype, void* workspace, int64_t workspace_bytes, hipStream_t stream);

// floats of one chunk image: per q-tile (16 heads) and 128-dim set, 8 float4 slots per lane, plus one
// slot per q-tile for (m, l); 64 lanes x 4 floats per slot
static inline int64_t part_image_floats(int64_t Hq, int64_t Hkv, int64_t Dv) {
  const int64_t qt = (Hq / Hkv + 15) / 16, ndv = (Dv + 127) / 128;
  return (qt * ndv * 8 + qt) * 256;
}

// bytes of workspace that is enough for any decode mode (the split form's chunk images)
int64_t vx_paged_attn_decode_workspace_bytes(int64_t num_seqs, int64_t Hq, int64_t Hkv, int64_t Dv,
                                             int64_t max_kv_len) {
  if (num_seqs <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || Dv <= 0 || max_kv_len <= 0) return 0;
  const int64_t nch = (max_kv_len + ATT_CHUNK - 1) / ATT_CHUNK;
  return num_seqs * Hkv * nch * part_image_floats(Hq, Hkv, Dv) * 4;
}

// bytes the launch with this mode will really use: 0 when it takes the fused form
int64_t vx_paged_attn_decode_workspace_needed(int64_t num_seqs, int64_t Hq, int64_t Hkv, int64_t Dv,
                                              int64_t max_kv_len, int mode) {
  if (mode != 0 && mode != 3 && mode != 4) return 0;
  if (num_seqs <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || Dv <= 0 || max_kv_len <= 0) return 0;
  if (decode_form(mode, num_seqs, (int)Hq, (int)Hkv, (int)Dv) == 1) return 0;
  return vx_paged_attn_decode_workspace_bytes(num_seqs, Hq, Hkv, Dv, max_kv_len);
}

// mode: 0 = paged decode (every sequence has <= 1 query token; needs workspace); 3 / 4 = the same,
//       forcing the split + combine kernels / the fused kernel (0 chooses; results are identical),
//       1 = paged general (prefill / mixed), 2 = packed K/V (cu_seqlens_k, no page table).
int vx_attention(const void* q, const void* k, const void* v, void* out, const int* cu_seqlens_q,
                 const int* seqused_k, const int* cu_seqlens_k, const int* block_table,
                 int64_t total_q, int64_t num_seqs, int Hq, int Hkv, int Dk, int Dv,
                 int64_t sqt, int64_t sqh, int64_t skb, int64_t skp, int64_t skh, int64_t svb,
                 int64_t svp, int64_t svh, int64_t sot, int64_t soh, int64_t bt_stride,
                 int64_t max_pages, int page_size, float softmax_scale, int causal, int mode,
                 int max_seqlen_q, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  return vx_attention_typed(q, k, v, out, nullptr, nullptr, cu_seqlens_q, seqused_k, cu_seqlens_k, block_table, total_q, num_seqs, Hq,
                            Hkv, Dk, Dv, sqt, sqh, skb, skp, skh, svb, svp, svh, sot, soh, bt_stride, max_pages, page_size,
                            softmax_scale, causal, mode, max_seqlen_q, 0, workspace, workspace_bytes, stream);
}

// vx_attention with two optional extras: lse [total_q, Hq] fp32 (natural log; modes 1 and 2 only) receives
// the rows' log-sum-exp, which the backward needs; seq_order [num_seqs] (paged modes) is a permutation
// of the sequences in which the decode kernels take them, e.g. longest context first (in a general launch it
// orders the decode kernel that takes the sequences of one query row).
int vx_attention_ex(const void* q, const void* k, const void* v, void* out, float* lse, const int* seq_order,
                    const int* cu_seqlens_q,
                     const int* seqused_k, const int* cu_seqlens_k, const int* block_table,
                     int64_t total_q, int64_t num_seqs, int Hq, int Hkv, int Dk, int Dv,
                     int64_t sqt, int64_t sqh, int64_t skb, int64_t skp, int64_t skh, int64_t svb,
                     int64_t svp, int64_t svh, int64_t sot, int64_t soh, int64_t bt_stride,
                     int64_t max_pages, int page_size, float softmax_scale, int causal, int mode,
                     int max_seqlen_q, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  return vx_attention_typed(q, k, v, out, lse, seq_order, cu_seqlens_q, seqused_k, cu_seqlens_k, block_table, total_q, num_seqs, Hq,
                            Hkv, Dk, Dv, sqt, sqh, skb, skp, skh, svb, svp, svh, sot, soh, bt_stride, max_pages, page_size,
                            softmax_scale, causal, mode, max_seqlen_q, 0, workspace, workspace_bytes, stream);
}

// vx_attention_ex for either 16-bit element type (dtype 0 = bf16, 1 = fp16; q, k, v and out share it) or fp32 (dtype 2:
// a correctness path of one thread per output row, attn_f32.h; no workspace, seq_order ignored) and any head sizes up to 256. bf16 at (Dk, Dv) in {(32, 32), (64, 64), (128, 128), (192, 128), (256, 256)} with 16-byte
// addressable rows runs the kernels built for exactly those sizes; everything else runs the kernels of the next
// built-for size with the missing query columns as zeros (same bits as an exact-size kernel would give), and
// per-element accesses when a head size or stride is not a multiple of 8 elements.
int vx_attention_typed(const void* q, const void* k, const void* v, void* out, float* lse, const int* seq_order,
                       const int* cu_seqlens_q, const int* seqused_k, const int* cu_seqlens_k, const int* block_table,
                       int64_t total_q, int64_t num_seqs, int Hq, int Hkv, int Dk, int Dv,
                       int64_t sqt, int64_t sqh, int64_t skb, int64_t skp, int64_t skh, int64_t svb,
                       int64_t svp, int64_t svh, int64_t sot, int64_t soh, int64_t bt_stride,
                       int64_t max_pages, int page_size, float softmax_scale, int causal, int mode,
                       int max_seqlen_q, int dtype, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  if (!q || !k || !v || !out || !cu_seqlens_q) return VX_ERR_ARG;
  if (dtype != 0 && dtype != 1 && dtype != 2) return VX_ERR_UNSUPPORTED;
  if (Dk <= 0 || Dv <= 0) return VX_ERR_ARG;
  if (Dk > 256 || Dv > 256) return VX_ERR_UNSUPPORTED;
  if (lse && mode != 1 && mode != 2) return VX_ERR_UNSUPPORTED;
  if (seq_order && mode == 2) return VX_ERR_UNSUPPORTED;
  if (total_q < 0 || num_seqs < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return VX_ERR_ARG;
  if (mode < 0 || mode > 4) return VX_ERR_ARG;
  if (mode != 2 && (!seqused_k || !block_table || page_size <= 0 || max_pages <= 0)) return VX_ERR_ARG;
  if (mode == 2 && !cu_seqlens_k) return VX_ERR_ARG;
  const bool decode = mode == 0 || mode == 3 || mode == 4;
  if (decode && !causal) return VX_ERR_UNSUPPORTED;
  if (total_q == 0 || num_seqs == 0) return VX_OK;
  if (num_seqs > 65535 || Hq > 65535) return VX_ERR_UNSUPPORTED;
  if (dtype == 2) {  // fp32: one thread per output row, the same routine for every mode (attn_f32.h)
    if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 4 != 0) return VX_ERR_ARG;
    AttnF32 f = {};
    f.q = (const float*)q; f.sqt = sqt; f.sqh = sqh;
    f.k = (const float*)k; f.skb = skb; f.skp = skp; f.skh = skh;
    f.v = (const float*)v; f.svb = svb; f.svp = svp; f.svh = svh;
    f.o = (float*)out; f.sot = sot; f.soh = soh;
    f.lse = lse;
    f.cu_q = cu_seqlens_q; f.seqused_k = seqused_k; f.cu_k = cu_seqlens_k;
    f.block_table = block_table; f.bt_stride = bt_stride;
    f.page_size = page_size;
    const int64_t mk = mode != 2 ? max_pages * (int64_t)page_size : 0;
    f.max_kv = (int)(mk > 0x7fffffff ? 0x7fffffff : mk);
    f.Hq = Hq; f.Hkv = Hkv; f.num_seqs = (int)num_seqs; f.dk = Dk; f.dv = Dv;
    f.causal = causal; f.packed = mode == 2 ? 1 : 0;
    f.scale = softmax_scale;
    return launch_attn_f32_forward(f, total_q, stream);
  }
  // rows that 16-byte accesses cannot address go element by element
  const bool elem = (sqt | sqh | skb | skp | skh | svb | svp | svh | sot | soh | (int64_t)Dk | (int64_t)Dv) % 8 != 0 ||
                    ((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 16 != 0;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 2 != 0) return VX_ERR_ARG;
  AttnParams p = {};
  p.dk = Dk; p.dv = Dv; p.elem = elem ? 1 : 0;
  p.q = (const bf16_t*)q; p.sqt = sqt; p.sqh = sqh;
  p.k = (const bf16_t*)k; p.skb = skb; p.skp = skp; p.skh = skh;
  p.v = (const bf16_t*)v; p.svb = svb; p.svp = svp; p.svh = svh;
  p.o = (bf16_t*)out; p.sot = sot; p.soh = soh;
  p.cu_q = cu_seqlens_q; p.seqused_k = seqused_k; p.cu_k = cu_seqlens_k;
  p.block_table = block_table; p.bt_stride = bt_stride;
  p.page_size = page_size;
  p.page_shift = -1;
  if (page_size > 0 && (page_size & (page_size - 1)) == 0) {
    int s = 0;
    while ((1 << s) < page_size) s++;
    p.page_shift = s;
  }
  p.Hq = Hq; p.Hkv = Hkv; p.num_seqs = (int)num_seqs;
  p.qk_scale = softmax_scale * 1.44269504f;
  p.causal = causal;
  p.lse = lse;
  p.seq_order = seq_order;
  {
    const int64_t mk = mode != 2 ? max_pages * (int64_t)page_size : 0;
    p.max_kv = (int)(mk > 0x7fffffff ? 0x7fffffff : mk);
  }
  if (decode) {
    const int64_t max_kv = max_pages * (int64_t)page_size;
    const int64_t nch = (max_kv + ATT_CHUNK - 1) / ATT_CHUNK;
    if (nch > 0x7fffffff) return VX_ERR_ARG;
    p.img_floats = part_image_floats(Hq, Hkv, Dv);
    p.max_chunks = (int)nch;
    if (decode_form(mode, num_seqs, Hq, Hkv, Dv) != 1) {  // the fused form keeps its chunk states in LDS
      const int64_t need = num_seqs * Hkv * nch * p.img_floats * 4;
      if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 15)) return VX_ERR_WORKSPACE;
      p.part = (float*)workspace;
    }
  }
  const int tq = (int)total_q;
  if (dtype == 0 && !elem) {
    if (Dk == 128 && Dv == 128) return launch_attn<ElemBF16, 128, 128, false>(p, mode, max_seqlen_q, tq, stream);
    if (Dk == 64 && Dv == 64) return launch_attn<ElemBF16, 64, 64, false>(p, mode, max_seqlen_q, tq, stream);
    if (Dk == 32 && Dv == 32) return launch_attn<ElemBF16, 32, 32, false>(p, mode, max_seqlen_q, tq, stream);
    if (Dk == 192 && Dv == 128) return launch_attn<ElemBF16, 192, 128, false>(p, mode, max_seqlen_q, tq, stream);
    if (Dk == 256 && Dv == 256) return launch_attn<ElemBF16, 256, 256, false>(p, mode, max_seqlen_q, tq, stream);
  }
  // the next built-for pair; the value size alone decides between one and two sets of output accumulators, which is
  // what the workspace and LDS figures above were computed from
  const int DVb = Dv > 128 ? 256 : (Dk > 64 || Dv > 64) ? 128 : 64;
  const int DKb = (Dk > 128 || DVb == 256) ? 256 : DVb;
  return dtype == 0 ? launch_attn_bf16_padded(p, DKb, DVb, mode, max_seqlen_q, tq, stream)
                    : launch_attn_f16(p, DKb, DVb, mode, max_seqlen_q, tq, stream);
}

// cache.view(-1, Hkv*D)[slot] = src[t]; value may be null (store one tensor only)
int vx_store_kvcache(const void* key, const void* value, void* k_cache, void* v_cache,
                     const int* slot_mapping, int64_t num_tokens, int64_t k_src_stride_bytes,
                     int64_t v_src_stride_bytes, int64_t k_row_bytes, int64_t v_row_bytes,
                     hipStream_t stream) {
  if (!key || !k_cache || !slot_mapping || num_tokens < 0) return VX_ERR_ARG;
  if (value && !v_cache) return VX_ERR_ARG;
  if (num_tokens == 0) return VX_OK;
  if (k_row_bytes % 16 != 0 || k_src_stride_bytes % 16 != 0 || k_row_bytes > 0x7fffffff) return VX_ERR_UNSUPPORTED;
  if (value && (v_row_bytes % 16 != 0 || v_src_stride_bytes % 16 != 0 || v_row_bytes > 0x7fffffff)) return VX_ERR_UNSUPPORTED;
  if (((uintptr_t)key | (uintptr_t)k_cache | (uintptr_t)value | (uintptr_t)v_cache) % 16 != 0) return VX_ERR_UNSUPPORTED;
  const int64_t blocks = (num_tokens + 3) / 4;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
  store_kv_kernel<<<(unsigned)blocks, 256, 0, stream>>>(
      (const uint8_t*)key, (const uint8_t*)value, (uint8_t*)k_cache, (uint8_t*)v_cache, slot_mapping,
      num_tokens, k_src_stride_bytes, v_src_stride_bytes, (int)k_row_bytes, (int)v_row_bytes);
  return launch_status();
}

int vx_store_kvcache_strided(const void* key, const void* value, void* k_cache, void* v_cache, const int* slot_mapping,
                             int64_t num_tokens, int heads, int64_t k_src_stride_bytes, int64_t v_src_stride_bytes,
                             int64_t k_head_bytes, int64_t v_head_bytes, int page_size, int64_t k_block_stride_bytes,
                             int64_t k_row_stride_bytes, int64_t k_head_stride_bytes, int64_t v_block_stride_bytes,
                             int64_t v_row_stride_bytes, int64_t v_head_stride_bytes, hipStream_t stream) {
  if (!key || !k_cache || !slot_mapping || num_tokens < 0 || heads <= 0 || page_size <= 0) return VX_ERR_ARG;
  if (value && !v_cache) return VX_ERR_ARG;
  if (num_tokens == 0) return VX_OK;
  if (k_head_bytes <= 0 || k_head_bytes % 16 != 0 || heads * k_head_bytes > 0x7fffffff) return VX_ERR_UNSUPPORTED;
  if ((k_src_stride_bytes | k_block_stride_bytes | k_row_stride_bytes | k_head_stride_bytes) % 16 != 0) return VX_ERR_UNSUPPORTED;
  if (value && (v_head_bytes <= 0 || v_head_bytes % 16 != 0 || heads * v_head_bytes > 0x7fffffff ||
                (v_src_stride_bytes | v_block_stride_bytes | v_row_stride_bytes | v_head_stride_bytes) % 16 != 0))
    return VX_ERR_UNSUPPORTED;
  if (((uintptr_t)key | (uintptr_t)k_cache | (uintptr_t)value | (uintptr_t)v_cache) % 16 != 0) return VX_ERR_UNSUPPORTED;
  const int64_t blocks = (num_tokens + 3) / 4;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
  store_kv_strided_kernel<<<(unsigned)blocks, 256, 0, stream>>>(
      (const uint8_t*)key, (const uint8_t*)value, (uint8_t*)k_cache, (uint8_t*)v_cache, slot_mapping, num_tokens,
      k_src_stride_bytes, v_src_stride_bytes, heads, (int)k_head_bytes, (int)v_head_bytes, page_size, k_block_stride_bytes,
      k_row_stride_bytes, k_head_stride_bytes, v_block_stride_bytes, v_row_stride_bytes, v_head_stride_bytes);
  return launch_status();
}

}  // extern "C"
