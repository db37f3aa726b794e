// fp32 attention, forward and backward: the third element type that the reference's kernels take
// (vexact/batch_invariant_ops/triton_invariant_attention.py:108-113, FP32_OUTPUT; its own backward tests run in
// fp32, tests/batch_invariant_ops/test_triton_attention_varlen.py:261-300, 335-395). No caller on the inference path
// uses it, so this is a correctness path, not a tuned one: one thread per output row, every sum a single ascending
// fp32 chain, true fp32 products (the reference's tl.dot would use TF32 here).
//
// Arithmetic per query row i of a sequence (keys 0 .. i + kv_len - q_len visible under the causal mask), c = scale * log2(e):
//   t_j = fl(s_j * c) with s_j = sum_d q_d k_jd (fused multiply-adds, d ascending) ; m = max_j t_j
//   p_j = exp2(fma(s_j, c, -m)) ; l = sum_j p_j ; out_d = (sum_j p_j v_jd) / l ; lse = (m + log2 l) ln 2
// A row's result depends on its own sequence only and is computed by the same routine whether the keys are packed or
// paged and whatever else is in the batch: batch invariant, and prefill, decode and packed results agree bit for bit.
// Backward (packed, causal), with P recomputed from the saved log-sum-exp as in the reference (:193-430):
//   delta_i = sum_d dO_id O_id ; p_ij = exp2(fma(s_ij, c, -lse_i log2 e)) ; dS_ij = p_ij (dO_i . v_j - delta_i) scale
//   dQ_i = sum_j dS_ij k_j ; dK_j = sum_{heads of the group, then rows i ascending} dS_ij q_i ; dV_j = sum p_ij dO_i
//
// Everything here is plain C++ with no device intrinsics, so the same functions can be compiled for the host by a test
// harness that checks arithmetic and addressing against the CPU oracle; the product only ever calls them from kernels.
#pragma once
#include <math.h>
#include <stdint.h>

namespace vx {

constexpr int ATT_F32_MAXD = 256;

struct AttnF32 {
  const float* q; int64_t sqt, sqh;         // [T, Hq, dk]
  const float* k; int64_t skb, skp, skh;    // paged: [blocks, page, Hkv, dk]; packed: [Tk, Hkv, dk], skp = row stride
  const float* v; int64_t svb, svp, svh;
  float* o; int64_t sot, soh;               // [T, Hq, dv]
  float* lse;                               // optional [T, Hq]
  const int* cu_q;                          // [num_seqs + 1]
  const int* seqused_k;                     // paged: [num_seqs]
  const int* cu_k;                          // packed: [num_seqs + 1]
  const int* block_table; int64_t bt_stride;
  int page_size, max_kv;                    // paged: keys that a block-table row can address
  int Hq, Hkv, num_seqs, dk, dv, causal, packed;
  float scale;
};

struct AttnF32Bwd {
  const float* q; int64_t sqt, sqh;
  const float* k; int64_t skt, skh;
  const float* v; int64_t svt, svh;
  const float* o; int64_t sot, soh;
  const float* d_o; int64_t sdt, sdh;
  const float* lse;                         // [T, Hq]
  float* delta;                             // [T, Hq] workspace
  float* dq; int64_t sdqt, sdqh;
  float* dk; int64_t sdkt, sdkh;
  float* dv; int64_t sdvt, sdvh;
  const int* cu_q; const int* cu_k;
  int Hq, Hkv, num_seqs, dk_, dv_;
  float scale;
};

// the sequence that packed row t belongs to: the last s with cu[s] <= t (empty sequences share their start with the
// next one and are skipped by "last")
__host__ __device__ inline int f32_seq_of(const int* cu, int num_seqs, int t) {
  int lo = 0, hi = num_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu[mid] <= t) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

__host__ __device__ inline float f32_dot(const float* a, const float* b, int n) {
  float s = 0.f;
  for (int d = 0; d < n; d++) s = fmaf(a[d], b[d], s);
  return s;
}

// row of key j (0-based inside the sequence) for kv head kvh; a page id below 0 (an unfilled table entry) reads page 0
__host__ __device__ inline const float* f32_kv_row(const AttnF32& p, const float* base, int64_t sb, int64_t sp, int64_t sh,
                                                   int seq, int k0, int j, int kvh) {
  if (p.packed) return base + (int64_t)(k0 + j) * sp + (int64_t)kvh * sh;
  int page = p.block_table[(int64_t)seq * p.bt_stride + j / p.page_size];
  if (page < 0) page = 0;
  return base + (int64_t)page * sb + (int64_t)(j % p.page_size) * sp + (int64_t)kvh * sh;
}

// output row of packed query row t, head h
__host__ __device__ inline void attn_f32_forward_row(const AttnF32& p, int t, int h) {
  const int seq = f32_seq_of(p.cu_q, p.num_seqs, t);
  const int q0 = p.cu_q[seq], qlen = p.cu_q[seq + 1] - q0, i = t - q0;
  if (i < 0 || i >= qlen) return;
  int k0 = 0, kv_len;
  if (p.packed) {
    k0 = p.cu_k[seq];
    kv_len = p.cu_k[seq + 1] - k0;
  } else {
    kv_len = p.seqused_k[seq];
    if (kv_len > p.max_kv) kv_len = p.max_kv;  // a wrong length must not walk off the block table
  }
  if (kv_len <= 0) return;  // a sequence without keys: its rows are left alone, as by the 16-bit kernels
  int visible = kv_len;
  if (p.causal) {
    const int last = i + (kv_len - qlen);
    visible = last + 1 < kv_len ? last + 1 : kv_len;
  }
  float* orow = p.o + (int64_t)t * p.sot + (int64_t)h * p.soh;
  float* lse = p.lse ? p.lse + (int64_t)t * p.Hq + h : nullptr;
  if (visible <= 0) {  // no visible key: the output is defined as 0, and +inf makes every recomputed probability 0
    for (int d = 0; d < p.dv; d++) orow[d] = 0.f;
    if (lse) *lse = INFINITY;
    return;
  }
  const int kvh = h / (p.Hq / p.Hkv);
  const float* qrow = p.q + (int64_t)t * p.sqt + (int64_t)h * p.sqh;
  const float c = p.scale * 1.44269504f;
  float m = -INFINITY;
  for (int j = 0; j < visible; j++) {
    const float s = f32_dot(qrow, f32_kv_row(p, p.k, p.skb, p.skp, p.skh, seq, k0, j, kvh), p.dk);
    m = fmaxf(m, s * c);
  }
  float acc[ATT_F32_MAXD];
  for (int d = 0; d < p.dv; d++) acc[d] = 0.f;
  float l = 0.f;
  for (int j = 0; j < visible; j++) {
    const float s = f32_dot(qrow, f32_kv_row(p, p.k, p.skb, p.skp, p.skh, seq, k0, j, kvh), p.dk);
    const float pj = exp2f(fmaf(s, c, -m));
    l += pj;
    const float* vrow = f32_kv_row(p, p.v, p.svb, p.svp, p.svh, seq, k0, j, kvh);
    for (int d = 0; d < p.dv; d++) acc[d] = fmaf(pj, vrow[d], acc[d]);
  }
  for (int d = 0; d < p.dv; d++) orow[d] = acc[d] / l;
  if (lse) *lse = (m + log2f(l)) * 0.6931471824645996f;
}

// delta of packed query row t, head h
__host__ __device__ inline void attn_f32_delta_row(const AttnF32Bwd& p, int t, int h) {
  p.delta[(int64_t)t * p.Hq + h] = f32_dot(p.d_o + (int64_t)t * p.sdt + (int64_t)h * p.sdh,
                                           p.o + (int64_t)t * p.sot + (int64_t)h * p.soh, p.dv_);
}

// dQ of packed query row t, head h
__host__ __device__ inline void attn_f32_dq_row(const AttnF32Bwd& p, int t, int h) {
  const int seq = f32_seq_of(p.cu_q, p.num_seqs, t);
  const int q0 = p.cu_q[seq], qlen = p.cu_q[seq + 1] - q0, i = t - q0;
  if (i < 0 || i >= qlen) return;
  const int k0 = p.cu_k[seq], kv_len = p.cu_k[seq + 1] - k0;
  float* dq = p.dq + (int64_t)t * p.sdqt + (int64_t)h * p.sdqh;
  float acc[ATT_F32_MAXD];
  for (int d = 0; d < p.dk_; d++) acc[d] = 0.f;
  const int last = i + (kv_len - qlen);
  const int visible = last + 1 < kv_len ? last + 1 : kv_len;
  if (visible > 0) {
    const int kvh = h / (p.Hq / p.Hkv);
    const float* qrow = p.q + (int64_t)t * p.sqt + (int64_t)h * p.sqh;
    const float* drow = p.d_o + (int64_t)t * p.sdt + (int64_t)h * p.sdh;
    const float c = p.scale * 1.44269504f;
    const float lse2 = p.lse[(int64_t)t * p.Hq + h] * 1.44269504f;
    const float delta = p.delta[(int64_t)t * p.Hq + h];
    for (int j = 0; j < visible; j++) {
      const float* krow = p.k + (int64_t)(k0 + j) * p.skt + (int64_t)kvh * p.skh;
      const float* vrow = p.v + (int64_t)(k0 + j) * p.svt + (int64_t)kvh * p.svh;
      const float pj = exp2f(fmaf(f32_dot(qrow, krow, p.dk_), c, -lse2));
      const float ds = pj * (f32_dot(drow, vrow, p.dv_) - delta) * p.scale;
      for (int d = 0; d < p.dk_; d++) acc[d] = fmaf(ds, krow[d], acc[d]);
    }
  }
  for (int d = 0; d < p.dk_; d++) dq[d] = acc[d];
}

// dK and dV of packed key row tk, kv head kvh: the query heads of the group in ascending order, each over the
// rows that see the key, ascending
__host__ __device__ inline void attn_f32_dkv_row(const AttnF32Bwd& p, int tk, int kvh) {
  const int seq = f32_seq_of(p.cu_k, p.num_seqs, tk);
  const int k0 = p.cu_k[seq], kv_len = p.cu_k[seq + 1] - k0, j = tk - k0;
  if (j < 0 || j >= kv_len) return;
  const int q0 = p.cu_q[seq], qlen = p.cu_q[seq + 1] - q0;
  float* dk = p.dk + (int64_t)tk * p.sdkt + (int64_t)kvh * p.sdkh;
  float* dv = p.dv + (int64_t)tk * p.sdvt + (int64_t)kvh * p.sdvh;
  float acck[ATT_F32_MAXD], accv[ATT_F32_MAXD];
  for (int d = 0; d < p.dk_; d++) acck[d] = 0.f;
  for (int d = 0; d < p.dv_; d++) accv[d] = 0.f;
  const float* krow = p.k + (int64_t)tk * p.skt + (int64_t)kvh * p.skh;
  const float* vrow = p.v + (int64_t)tk * p.svt + (int64_t)kvh * p.svh;
  const float c = p.scale * 1.44269504f;
  const int G = p.Hq / p.Hkv;
  int first = j - (kv_len - qlen);  // row i sees key j when j <= i + kv_len - qlen
  if (first < 0) first = 0;
  for (int gidx = 0; gidx < G; gidx++) {
    const int h = kvh * G + gidx;
    for (int i = first; i < qlen; i++) {
      const int64_t t = q0 + i;
      const float* qrow = p.q + t * p.sqt + (int64_t)h * p.sqh;
      const float* drow = p.d_o + t * p.sdt + (int64_t)h * p.sdh;
      const float lse2 = p.lse[t * p.Hq + h] * 1.44269504f;
      const float pj = exp2f(fmaf(f32_dot(qrow, krow, p.dk_), c, -lse2));
      const float ds = pj * (f32_dot(drow, vrow, p.dv_) - p.delta[t * p.Hq + h]) * p.scale;
      for (int d = 0; d < p.dv_; d++) accv[d] = fmaf(pj, drow[d], accv[d]);
      for (int d = 0; d < p.dk_; d++) acck[d] = fmaf(ds, qrow[d], acck[d]);
    }
  }
  for (int d = 0; d < p.dk_; d++) dk[d] = acck[d];
  for (int d = 0; d < p.dv_; d++) dv[d] = accv[d];
}

}  // namespace vx
