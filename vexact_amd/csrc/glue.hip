// Glue between the hot-path kernels of a Qwen3-style decoder layer, fused so that a decode
// step is a short, capture-safe launch sequence:
//   * vx_qk_norm_rope_store : per-head RMSNorm of q and k (two-rounding HuggingFace form), rotary
//     embedding in bf16, q written out, k and v scattered into the paged cache at slot_mapping
//     (the scatter is what store_kvcache does, vexact/batch_invariant_ops/kv_cache_context.py:294-314)
//   * vx_embedding          : row gather
//   * vx_fill_i32           : small fill kernel (graph-safe replacement for a memset node)
// The per-head sum of squares uses the same lane ownership and butterfly as the 64-thread
// variant of vx_rms_norm, so fused and unfused paths give the same bits.
#include "common.h"
#include <math.h>

namespace vx {

// grid = (ceil(T*(Hq+2Hkv)/8)); half a wavefront per (token, head): 32 lanes, lane l < D/4 of the
// half owns elements 4l .. 4l+3. qkv row layout: [q heads | k heads | v heads], each head D wide.
// The sum of squares is a 5-step butterfly inside the half: the same additions, in the same order, as a
// 64-lane butterfly whose upper 32 lanes hold zeros.
template <int D, typename PosT>
__global__ __launch_bounds__(256) void qk_norm_rope_store_kernel(
    const bf16_t* __restrict__ qkv, int64_t ld, const bf16_t* __restrict__ qw,
    const bf16_t* __restrict__ kw, const bf16_t* __restrict__ cos_t, const bf16_t* __restrict__ sin_t,
    const PosT* __restrict__ positions, const int* __restrict__ slots, bf16_t* __restrict__ q_out,
    bf16_t* __restrict__ k_out, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int64_t T,
    int Hq, int Hkv, float eps, int64_t max_pos, int page_size, int64_t csb, int64_t csp, int64_t csh) {
  const int HT = Hq + 2 * Hkv;
  const int64_t wid = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);  // (token, head) item of this half wavefront
  if (wid >= T * HT) return;
  const int64_t t = wid / HT;
  const int h = (int)(wid % HT);
  const int lane = threadIdx.x & 31;          // lane inside the half
  const int half_base = threadIdx.x & 32;     // first lane of the half inside the wavefront
  const bool own = lane < D / 4;
  const bf16_t* src = qkv + t * ld + (int64_t)h * D;
  uint2 raw = make_uint2(0, 0);
  if (own) raw = *(const uint2*)(src + 4 * lane);
  const int slot = slots ? slots[t] : -1;
  // cache element offset of this token's row: block slot / page, in-page row slot % page
  const int64_t crow = slot >= 0 ? (int64_t)(slot / page_size) * csb + (int64_t)(slot % page_size) * csp : 0;
  if (h >= Hq + Hkv) {  // value head: plain copy into the cache
    if (own && slot >= 0 && v_cache)
      *(uint2*)(v_cache + crow + (int64_t)(h - Hq - Hkv) * csh + 4 * lane) = raw;
    return;
  }
  // position, norm weight and rotary rows are requested before the reduction so that their
  // latency overlaps it
  const bf16_t* w = (h < Hq) ? qw : kw;
  int64_t pos = positions ? (int64_t)positions[t] : t;  // no positions: row t of the tables belongs to token t
  pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
  uint2 wr = make_uint2(0, 0), cr = make_uint2(0, 0), sr = make_uint2(0, 0);
  if (own) {
    wr = *(const uint2*)(w + 4 * lane);
    cr = *(const uint2*)(cos_t + pos * D + 4 * lane);
    sr = *(const uint2*)(sin_t + pos * D + 4 * lane);
  }
  float x[4] = {bf16lo(raw.x), bf16hi(raw.x), bf16lo(raw.y), bf16hi(raw.y)};
  float acc = 0.f;
  if (own) {
#pragma unroll
    for (int c = 0; c < 4; c++) acc += x[c] * x[c];
  }
  float tot = acc;
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) tot += __shfl_xor(tot, o, 64);
  const float inv = rms_inv(tot / (float)D + eps, 1);  // HuggingFace's q / k norm
  float y[4], cs[4], sn[4];
  if (own) {
    const float wf[4] = {bf16lo(wr.x), bf16hi(wr.x), bf16lo(wr.y), bf16hi(wr.y)};
    cs[0] = bf16lo(cr.x); cs[1] = bf16hi(cr.x); cs[2] = bf16lo(cr.y); cs[3] = bf16hi(cr.y);
    sn[0] = bf16lo(sr.x); sn[1] = bf16hi(sr.x); sn[2] = bf16lo(sr.y); sn[3] = bf16hi(sr.y);
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const float tn = bf16_to_f32(f32_to_bf16(x[c] * inv));
      y[c] = bf16_to_f32(f32_to_bf16(wf[c] * tn));
    }
  } else {
#pragma unroll
    for (int c = 0; c < 4; c++) { y[c] = 0.f; cs[c] = 0.f; sn[c] = 0.f; }
  }
  // rotate_half partner: element j pairs with j + D/2 (first half gets -partner)
  constexpr int HL = D / 8;  // lanes per half
  const bool first = lane < HL;
  float o[4];
#pragma unroll
  for (int c = 0; c < 4; c++) {
    const float partner = __shfl(y[c], half_base + (first ? lane + HL : lane - HL), 64);
    const float rot = first ? -partner : partner;
    const float a = bf16_to_f32(f32_to_bf16(y[c] * cs[c]));
    const float b = bf16_to_f32(f32_to_bf16(rot * sn[c]));
    o[c] = a + b;
  }
  if (!own) return;
  uint2 pk;
  pk.x = pack_bf16x2(o[0], o[1]);
  pk.y = pack_bf16x2(o[2], o[3]);
  if (h < Hq) {
    *(uint2*)(q_out + (t * Hq + h) * D + 4 * lane) = pk;
  } else {
    const int kh = h - Hq;
    if (k_out) *(uint2*)(k_out + (t * Hkv + kh) * D + 4 * lane) = pk;
    if (slot >= 0 && k_cache) *(uint2*)(k_cache + crow + (int64_t)kh * csh + 4 * lane) = pk;
  }
}

template <typename IdT>
__global__ __launch_bounds__(256) void embedding_kernel(const bf16_t* __restrict__ table,
                                                        const IdT* __restrict__ ids,
                                                        bf16_t* __restrict__ out, int64_t T, int H,
                                                        int64_t vocab) {
  const int64_t t = blockIdx.x;
  int64_t id = (int64_t)ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const uint4* src = (const uint4*)(table + id * H);
  uint4* dst = (uint4*)(out + t * H);
  for (int c = threadIdx.x; c < H / 8; c += 256) dst[c] = src[c];
}

// Rotary embedding of [T, H, D] rows from per-token cos / sin rows [T, D], HuggingFace's apply_rotary_pos_emb:
// out = r16(r16(x cos) + r16(rotate_half(x) sin)), rotate_half(x) = (-x[D/2:], x[:D/2]). One thread per group of
// 4 elements of the first half and their 4 partners in the second half.
__global__ __launch_bounds__(256) void rope_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ out,
                                                   const bf16_t* __restrict__ cos_r, const bf16_t* __restrict__ sin_r,
                                                   int64_t items, int H, int D, int64_t sxt, int64_t sxh, int64_t sot,
                                                   int64_t soh, int64_t scs) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= items) return;
  const int per = D / 8;  // threads per (token, head)
  const int c4 = (int)(i % per) * 4;
  const int64_t th = i / per;
  const int h = (int)(th % H);
  const int64_t t = th / H;
  const bf16_t* xp = x + t * sxt + (int64_t)h * sxh;
  const uint2 a = *(const uint2*)(xp + c4), b = *(const uint2*)(xp + D / 2 + c4);
  const uint2 ca = *(const uint2*)(cos_r + t * scs + c4), cb = *(const uint2*)(cos_r + t * scs + D / 2 + c4);
  const uint2 sa = *(const uint2*)(sin_r + t * scs + c4), sb = *(const uint2*)(sin_r + t * scs + D / 2 + c4);
  const float x1[4] = {bf16lo(a.x), bf16hi(a.x), bf16lo(a.y), bf16hi(a.y)};
  const float x2[4] = {bf16lo(b.x), bf16hi(b.x), bf16lo(b.y), bf16hi(b.y)};
  const float c1[4] = {bf16lo(ca.x), bf16hi(ca.x), bf16lo(ca.y), bf16hi(ca.y)};
  const float c2[4] = {bf16lo(cb.x), bf16hi(cb.x), bf16lo(cb.y), bf16hi(cb.y)};
  const float s1[4] = {bf16lo(sa.x), bf16hi(sa.x), bf16lo(sa.y), bf16hi(sa.y)};
  const float s2[4] = {bf16lo(sb.x), bf16hi(sb.x), bf16lo(sb.y), bf16hi(sb.y)};
  float o1[4], o2[4];
#pragma unroll
  for (int c = 0; c < 4; c++) {
    o1[c] = bf16_to_f32(f32_to_bf16(x1[c] * c1[c])) + bf16_to_f32(f32_to_bf16(-x2[c] * s1[c]));
    o2[c] = bf16_to_f32(f32_to_bf16(x2[c] * c2[c])) + bf16_to_f32(f32_to_bf16(x1[c] * s2[c]));
  }
  bf16_t* op = out + t * sot + (int64_t)h * soh;
  *(uint2*)(op + c4) = make_uint2(pack_bf16x2(o1[0], o1[1]), pack_bf16x2(o1[2], o1[3]));
  *(uint2*)(op + D / 2 + c4) = make_uint2(pack_bf16x2(o2[0], o2[1]), pack_bf16x2(o2[2], o2[3]));
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int* p, int v, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = v;
}

}  // namespace vx

using namespace vx;

extern "C" {

int vx_qk_norm_rope_store(const void* qkv, int64_t ld, const void* q_norm_w, const void* k_norm_w,
                          const void* cos_table, const void* sin_table, const void* positions,
                          int pos_i64, const int* slot_mapping, void* q_out, void* k_out,
                          void* k_cache, void* v_cache, int64_t T, int Hq, int Hkv, int D, float eps,
                          int64_t max_pos, int page_size, int64_t cache_block_stride,
                          int64_t cache_row_stride, int64_t cache_head_stride, hipStream_t stream) {
  if (!qkv || !q_norm_w || !k_norm_w || !cos_table || !sin_table || !q_out) return VX_ERR_ARG;
  if (T < 0 || Hq <= 0 || Hkv <= 0 || max_pos <= 0) return VX_ERR_ARG;
  if (D != 128 && D != 64) return VX_ERR_UNSUPPORTED;
  if (ld % 4 != 0) return VX_ERR_UNSUPPORTED;
  if (k_cache || v_cache) {
    if (page_size <= 0) return VX_ERR_ARG;
    if (cache_block_stride % 4 != 0 || cache_row_stride % 4 != 0 || cache_head_stride % 4 != 0)
      return VX_ERR_UNSUPPORTED;
  } else {
    page_size = 1;
  }
  if (T == 0) return VX_OK;
  const int64_t items = T * (Hq + 2 * Hkv);
  const int64_t blocks = (items + 7) / 8;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
#define VX_QK(DD, PT)                                                                          \
  qk_norm_rope_store_kernel<DD, PT><<<(unsigned)blocks, 256, 0, stream>>>(                     \
      (const bf16_t*)qkv, ld, (const bf16_t*)q_norm_w, (const bf16_t*)k_norm_w,                \
      (const bf16_t*)cos_table, (const bf16_t*)sin_table, (const PT*)positions, slot_mapping,  \
      (bf16_t*)q_out, (bf16_t*)k_out, (bf16_t*)k_cache, (bf16_t*)v_cache, T, Hq, Hkv, eps, max_pos,     \
      page_size, cache_block_stride, cache_row_stride, cache_head_stride)
  if (D == 128) { if (pos_i64) VX_QK(128, int64_t); else VX_QK(128, int); }
  else { if (pos_i64) VX_QK(64, int64_t); else VX_QK(64, int); }
#undef VX_QK
  return launch_status();
}

int vx_rope(const void* x, void* out, const void* cos_rows, const void* sin_rows, int64_t T, int H, int D,
            int64_t x_token_stride, int64_t x_head_stride, int64_t out_token_stride, int64_t out_head_stride,
            int64_t cos_row_stride, hipStream_t stream) {
  if (!x || !out || !cos_rows || !sin_rows || T < 0 || H <= 0 || D <= 0) return VX_ERR_ARG;
  if (D % 8 != 0) return VX_ERR_UNSUPPORTED;
  if ((x_token_stride | x_head_stride | out_token_stride | out_head_stride | cos_row_stride) % 4 != 0) return VX_ERR_UNSUPPORTED;
  if (((uintptr_t)x | (uintptr_t)out | (uintptr_t)cos_rows | (uintptr_t)sin_rows) % 8 != 0) return VX_ERR_UNSUPPORTED;
  if (T == 0) return VX_OK;
  const int64_t items = T * H * (D / 8);
  const int64_t blocks = (items + 255) / 256;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
  rope_kernel<<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, (const bf16_t*)cos_rows,
                                                    (const bf16_t*)sin_rows, items, H, D, x_token_stride, x_head_stride,
                                                    out_token_stride, out_head_stride, cos_row_stride);
  return launch_status();
}

int vx_embedding(const void* table, const void* ids, int ids_i64, void* out, int64_t T, int64_t H,
                 int64_t vocab, hipStream_t stream) {
  if (!table || !ids || !out || T < 0 || H <= 0 || vocab <= 0) return VX_ERR_ARG;
  if (H % 8 != 0 || H > 0x7fffffff) return VX_ERR_UNSUPPORTED;
  if (T == 0) return VX_OK;
  if (T > 0x7fffffffLL) return VX_ERR_ARG;
  if (ids_i64)
    embedding_kernel<int64_t><<<(unsigned)T, 256, 0, stream>>>((const bf16_t*)table, (const int64_t*)ids,
                                                               (bf16_t*)out, T, (int)H, vocab);
  else
    embedding_kernel<int><<<(unsigned)T, 256, 0, stream>>>((const bf16_t*)table, (const int*)ids,
                                                           (bf16_t*)out, T, (int)H, vocab);
  return launch_status();
}

int vx_fill_i32(int* p, int value, int64_t n, hipStream_t stream) {
  if (!p || n < 0) return VX_ERR_ARG;
  if (n == 0) return VX_OK;
  const int64_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
  fill_i32_kernel<<<(unsigned)blocks, 256, 0, stream>>>(p, value, n);
  return launch_status();
}

const char* vx_status_string(int code) {
  switch (code) {
    case VX_OK: return "ok";
    case VX_ERR_ARG: return "invalid argument (null pointer, negative size or bad stride)";
    case VX_ERR_UNSUPPORTED: return "unsupported shape, dtype, alignment or layout";
    case VX_ERR_WORKSPACE: return "workspace too small";
    case VX_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
  }
}

int vx_abi_version() { return 8; }

}  // extern "C"
