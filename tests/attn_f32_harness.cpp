// Host build of the fp32 attention routines (vexact_amd/csrc/attn_f32.h), for tests only: the row functions that
// the kernels call, driven by plain loops over the (row, head) indices that the kernels derive from their thread ids.
// Compiled by tests/test_attn_f32_host.py with g++; nothing in the product uses it.
#define __host__
#define __device__
#include "../vexact_amd/csrc/attn_f32.h"

extern "C" {

// ints: Hq, Hkv, num_seqs, dk, dv, causal, packed, page_size, max_kv, total_q
// strides (elements): sqt, sqh, skb, skp, skh, svb, svp, svh, sot, soh, bt_stride
void f32_forward(const float* q, const float* k, const float* v, float* o, float* lse, const int* cu_q,
                 const int* seqused_k, const int* cu_k, const int* block_table, const int* ints,
                 const int64_t* strides, float scale) {
  vx::AttnF32 p = {};
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
  p.cu_q = cu_q; p.seqused_k = seqused_k; p.cu_k = cu_k; p.block_table = block_table;
  p.Hq = ints[0]; p.Hkv = ints[1]; p.num_seqs = ints[2]; p.dk = ints[3]; p.dv = ints[4];
  p.causal = ints[5]; p.packed = ints[6]; p.page_size = ints[7]; p.max_kv = ints[8];
  p.sqt = strides[0]; p.sqh = strides[1]; p.skb = strides[2]; p.skp = strides[3]; p.skh = strides[4];
  p.svb = strides[5]; p.svp = strides[6]; p.svh = strides[7]; p.sot = strides[8]; p.soh = strides[9];
  p.bt_stride = strides[10];
  p.scale = scale;
  const int64_t n = (int64_t)ints[9] * p.Hq;
  for (int64_t idx = 0; idx < n; idx++) vx::attn_f32_forward_row(p, (int)(idx / p.Hq), (int)(idx % p.Hq));
}

// ints: Hq, Hkv, num_seqs, dk, dv, total_q, total_k; strides: token and head strides of q, k, v, out, dout, dq, dk, dv
void f32_backward(const float* q, const float* k, const float* v, const float* o, const float* d_o, const float* lse,
                  float* delta, float* dq, float* dk, float* dv, const int* cu_q, const int* cu_k, const int* ints,
                  const int64_t* s, float scale) {
  vx::AttnF32Bwd p = {};
  p.q = q; p.k = k; p.v = v; p.o = o; p.d_o = d_o; p.lse = lse; p.delta = delta; p.dq = dq; p.dk = dk; p.dv = dv;
  p.sqt = s[0]; p.sqh = s[1]; p.skt = s[2]; p.skh = s[3]; p.svt = s[4]; p.svh = s[5]; p.sot = s[6]; p.soh = s[7];
  p.sdt = s[8]; p.sdh = s[9]; p.sdqt = s[10]; p.sdqh = s[11]; p.sdkt = s[12]; p.sdkh = s[13]; p.sdvt = s[14]; p.sdvh = s[15];
  p.cu_q = cu_q; p.cu_k = cu_k;
  p.Hq = ints[0]; p.Hkv = ints[1]; p.num_seqs = ints[2]; p.dk_ = ints[3]; p.dv_ = ints[4];
  p.scale = scale;
  const int64_t nq = (int64_t)ints[5] * p.Hq, nk = (int64_t)ints[6] * p.Hkv;
  for (int64_t idx = 0; idx < nq; idx++) vx::attn_f32_delta_row(p, (int)(idx / p.Hq), (int)(idx % p.Hq));
  for (int64_t idx = 0; idx < nq; idx++) vx::attn_f32_dq_row(p, (int)(idx / p.Hq), (int)(idx % p.Hq));
  for (int64_t idx = 0; idx < nk; idx++) vx::attn_f32_dkv_row(p, (int)(idx / p.Hkv), (int)(idx % p.Hkv));
}

}  // extern "C"
