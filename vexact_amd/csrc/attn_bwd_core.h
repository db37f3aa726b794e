// Generic (register-form) kernels of the attention backward, for either 16-bit element type and any head sizes up
// to 256: included by attn_bwd.hip (bf16) and attn_bwd_f16.hip (fp16). See attn_bwd.hip for the formulas.
#pragma once
#include <algorithm>

#include "attn_core.h"

namespace vx {

struct AttnBwdParams {
  const bf16_t *q, *k, *v, *o, *d_o;
  const float* lse;  // [T, Hq] natural log
  float* delta;      // [T, Hq] workspace
  bf16_t *dq, *dk, *dv;
  int64_t sqt, sqh, skt, skh, svt, svh, sot, soh, sdt, sdh, sdqt, sdqh, sdkt, sdkh, sdvt, sdvh;
  const int *cu_q, *cu_k;
  int Hq, Hkv, num_seqs;
  float scale;
  int dk_, dv_, elem;  // head sizes of q / k and of v / out / dout as the caller has them; elem: see AttnParams
};

// delta[t, h] = sum_d f32(O[t, h, d]) f32(dO[t, h, d]): 16 lanes per (token, head) row, 8 dims each per 128 dims,
// then a fixed butterfly over the 16 lanes
template <class ET, int D, bool PAD>
__global__ __launch_bounds__(256) void attn_bwd_delta_kernel(AttnBwdParams p, int64_t total_q) {
  const int64_t i = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int c = threadIdx.x & 15;
  const bool live = i < total_q * p.Hq;
  const int64_t ii = live ? i : 0;
  const int64_t t = ii / p.Hq;
  const int h = (int)(ii % p.Hq);
  const int dv = PAD ? p.dv_ : D, elem = PAD ? p.elem : 0;
  float s = 0.f;
#pragma unroll
  for (int col = 0; col < D; col += 128) {
    if (col + 8 * c < dv) {
      const uint4 a = attn_ld8<PAD>(p.o + t * p.sot + (int64_t)h * p.soh, col + 8 * c, dv, elem);
      const uint4 b = attn_ld8<PAD>(p.d_o + t * p.sdt + (int64_t)h * p.sdh, col + 8 * c, dv, elem);
      s += ET::lo(a.x) * ET::lo(b.x); s += ET::hi(a.x) * ET::hi(b.x);
      s += ET::lo(a.y) * ET::lo(b.y); s += ET::hi(a.y) * ET::hi(b.y);
      s += ET::lo(a.z) * ET::lo(b.z); s += ET::hi(a.z) * ET::hi(b.z);
      s += ET::lo(a.w) * ET::lo(b.w); s += ET::hi(a.w) * ET::hi(b.w);
    }
  }
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
  if (live && c == 0) p.delta[i] = s;
}

// The moving rows of a 64-row block in the layout the transposed products read, for the 128 dims of set ds: slot idx
// of half ch holds row 32 ch + 16 (idx / 4) + 4 g + idx % 4, dims 128 ds + 8 r16 .. +8 (16 lanes cover 256 bytes of a
// row). rowp(r) = pointer to moving row r of the block, clamped to an existing row (its weight is 0). d: valid dims.
template <bool PAD, class RowPtr>
__device__ __forceinline__ void bwd_tr_load(RowPtr rowp, int ds, int d, int elem, uint4 (&rows)[2][8]) {
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int col = 128 * ds + 8 * r16;
#pragma unroll
  for (int ch = 0; ch < 2; ch++)
#pragma unroll
    for (int idx = 0; idx < 8; idx++) {
      const int r = 32 * ch + 16 * (idx >> 2) + 4 * g + (idx & 3);
      if constexpr (PAD) rows[ch][idx] = attn_ld8<true>(rowp(r), col, d, elem);
      else rows[ch][idx] = ldg16_raw(rowp(r) + (col < d ? col : 0));
    }
}

// acc[td] (rows = dims 128 ds + 8 r16' + td, cols = stationary) += (moving rows 0..63, transposed) x pf
template <class ET>
__device__ __forceinline__ void bwd_tr_product(const uint4 (&rows)[2][8], int ds, int d, const uint4 (&pf)[2], f32x4 (&acc)[8]) {
  const int r16 = threadIdx.x & 15;
  const bool dok = 128 * ds + 8 * r16 < d;
#pragma unroll
  for (int ch = 0; ch < 2; ch++) {
#pragma unroll
    for (int td = 0; td < 8; td++) {
      uint32_t w[4];
#pragma unroll
      for (int qd = 0; qd < 4; qd++) {
        const uint4 ra = mask16(rows[ch][2 * qd], dok), rb = mask16(rows[ch][2 * qd + 1], dok);
        const uint32_t a = (td < 2) ? ra.x : (td < 4) ? ra.y : (td < 6) ? ra.z : ra.w;
        const uint32_t b = (td < 2) ? rb.x : (td < 4) ? rb.y : (td < 6) ? rb.z : rb.w;
        w[qd] = (td & 1) ? ((a >> 16) | (b & 0xffff0000u)) : ((a & 0xffffu) | (b << 16));
      }
      acc[td] = ET::mfma(make_uint4(w[0], w[1], w[2], w[3]), pf[ch], acc[td]);
    }
  }
}

// lane (g, c) holds acc[td][r] = element (dim 128 ds + 32 g + 8 r + td) of stationary row c: 16 bytes per r
template <class ET, bool PAD>
__device__ __forceinline__ void bwd_store_tile(const f32x4 (&acc)[8], int ds, int d, int elem, bf16_t* rowp) {
  const int g = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int d0 = 128 * ds + 32 * g + 8 * r;
    if (d0 >= d) continue;
    uint4 pk;
    pk.x = ET::pack2(acc[0][r], acc[1][r]);
    pk.y = ET::pack2(acc[2][r], acc[3][r]);
    pk.z = ET::pack2(acc[4][r], acc[5][r]);
    pk.w = ET::pack2(acc[6][r], acc[7][r]);
    attn_st8<PAD>(rowp, d0, pk, d, elem);
  }
}

template <class ET>
__device__ __forceinline__ void bwd_pack(const float (&x)[4][4], uint4 (&pf)[2]) {
  uint32_t pw[4][2];
#pragma unroll
  for (int tt = 0; tt < 4; tt++) {
    pw[tt][0] = ET::pack2(x[tt][0], x[tt][1]);
    pw[tt][1] = ET::pack2(x[tt][2], x[tt][3]);
  }
  pf[0] = make_uint4(pw[0][0], pw[0][1], pw[1][0], pw[1][1]);
  pf[1] = make_uint4(pw[2][0], pw[2][1], pw[3][0], pw[3][1]);
}

// fragment of a row for a score product: dims 32 s + 8 g .. +8, zeros past d when `zero` (the stationary side and
// one side of every product must carry the zeros; the other side may then hold anything finite there)
template <bool PAD>
__device__ __forceinline__ uint4 bwd_frag(const bf16_t* row, int s, int d, int elem, bool zero) {
  const int g = (threadIdx.x & 63) >> 4, col = 32 * s + 8 * g;
  const uint4 v = attn_ld8<PAD>(row, col, d, elem);
  if constexpr (PAD) return zero ? mask16(v, col < d) : v;
  return v;
}

// ---- dQ: grid (query tiles / 4, Hq, sequences), wavefront = 16 queries of one head ------------
// D: built-for head size (both q / k and v); up to 128 every load of a block is issued before the first is used (one
// memory round trip per block), above that the fragments of one 16-key tile at a time (registers).
template <class ET, int D, bool PAD>
__global__ __launch_bounds__(256) void attn_bwd_dq_kernel(AttnBwdParams p) {
  constexpr int KS = D / 32, NDS = (D + 127) / 128;
  constexpr bool HOIST = D <= 128;
  const int dk = PAD ? p.dk_ : D, dv = PAD ? p.dv_ : D, elem = PAD ? p.elem : 0;
  const int seq = blockIdx.z, h = blockIdx.y;
  const int q0 = p.cu_q[seq], qlen = p.cu_q[seq + 1] - q0;
  const int k0 = p.cu_k[seq], kv_len = p.cu_k[seq + 1] - k0;
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int i0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 16;
  if (i0 >= qlen || kv_len <= 0) return;
  const int kvh = h / (p.Hq / p.Hkv);
  const int shift = kv_len - qlen;
  const int i = i0 + r16;                      // this lane's query (stationary column)
  const bool qok = i < qlen;
  const int pos = qok ? shift + i : -1;        // last visible key; -1: nothing visible
  const int64_t tq = q0 + (qok ? i : qlen - 1);
  uint4 qf[KS], of[KS];
  {
    const bf16_t* qp = p.q + tq * p.sqt + (int64_t)h * p.sqh;
    const bf16_t* dp = p.d_o + tq * p.sdt + (int64_t)h * p.sdh;
#pragma unroll
    for (int s = 0; s < KS; s++) {
      qf[s] = bwd_frag<PAD>(qp, s, dk, elem, true);
      of[s] = bwd_frag<PAD>(dp, s, dv, elem, true);
    }
  }
  const float c2 = p.scale * 1.44269504f;
  const float lse2 = p.lse[tq * p.Hq + h] * 1.44269504f;
  const float delta = p.delta[tq * p.Hq + h];
  int maxpos = pos;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) maxpos = max(maxpos, __shfl_xor(maxpos, o, 64));
  maxpos = min(maxpos, kv_len - 1);

  f32x4 acc[NDS][8];
#pragma unroll
  for (int ds = 0; ds < NDS; ds++)
#pragma unroll
    for (int td = 0; td < 8; td++) acc[ds][td] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16_t* kb_ = p.k + (int64_t)k0 * p.skt + (int64_t)kvh * p.skh;
  const bf16_t* vb_ = p.v + (int64_t)k0 * p.svt + (int64_t)kvh * p.svh;
  for (int kb = 0; kb <= maxpos; kb += 64) {
    uint4 kfr[HOIST ? 4 : 1][KS], vfr[HOIST ? 4 : 1][KS], rows[2][8];
    auto load_tile = [&](int tt, int slot) {
      const int64_t kr = min(kb + 16 * tt + r16, kv_len - 1);
#pragma unroll
      for (int s = 0; s < KS; s++) {
        kfr[slot][s] = bwd_frag<PAD>(kb_ + kr * p.skt, s, dk, elem, false);
        vfr[slot][s] = bwd_frag<PAD>(vb_ + kr * p.svt, s, dv, elem, false);
      }
    };
    if constexpr (HOIST) {
#pragma unroll
      for (int tt = 0; tt < 4; tt++) load_tile(tt, tt);
      bwd_tr_load<PAD>([&](int r) { return kb_ + (int64_t)min(kb + r, kv_len - 1) * p.skt; }, 0, dk, elem, rows);
    }
    float ds_[4][4];
#pragma unroll
    for (int tt = 0; tt < 4; tt++) {
      if constexpr (!HOIST) load_tile(tt, 0);
      const int slot = HOIST ? tt : 0;
      f32x4 st = f32x4{0.f, 0.f, 0.f, 0.f}, dp = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; s++) {
        st = ET::mfma(kfr[slot][s], qf[s], st);
        dp = ET::mfma(vfr[slot][s], of[s], dp);
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int key = kb + 16 * tt + 4 * g + r;
        const float pr = (key <= pos) ? __builtin_amdgcn_exp2f(__builtin_fmaf(st[r], c2, -lse2)) : 0.f;
        ds_[tt][r] = pr * (dp[r] - delta) * p.scale;
      }
    }
    uint4 pf[2];
    bwd_pack<ET>(ds_, pf);
#pragma unroll
    for (int ds = 0; ds < NDS; ds++) {
      if (!HOIST || ds > 0)
        bwd_tr_load<PAD>([&](int r) { return kb_ + (int64_t)min(kb + r, kv_len - 1) * p.skt; }, ds, dk, elem, rows);
      bwd_tr_product<ET>(rows, ds, dk, pf, acc[ds]);
    }
  }
  if (qok) {
#pragma unroll
    for (int ds = 0; ds < NDS; ds++) bwd_store_tile<ET, PAD>(acc[ds], ds, dk, elem, p.dq + tq * p.sdqt + (int64_t)h * p.sdqh);
  }
}

// ---- dK, dV: grid (key tiles / 4, Hkv, sequences), wavefront = 16 keys of one kv head ----------
template <class ET, int D, bool PAD>
__global__ __launch_bounds__(256) void attn_bwd_dkv_kernel(AttnBwdParams p) {
  constexpr int KS = D / 32, NDS = (D + 127) / 128;
  constexpr bool HOIST = D <= 128;
  const int dk_n = PAD ? p.dk_ : D, dv_n = PAD ? p.dv_ : D, elem = PAD ? p.elem : 0;
  const int seq = blockIdx.z, kvh = blockIdx.y;
  const int q0 = p.cu_q[seq], qlen = p.cu_q[seq + 1] - q0;
  const int k0 = p.cu_k[seq], kv_len = p.cu_k[seq + 1] - k0;
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int j0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 16;
  if (j0 >= kv_len) return;
  const int G = p.Hq / p.Hkv;
  const int shift = kv_len - qlen;
  const int j = j0 + r16;                       // this lane's key (stationary column)
  const bool kok = j < kv_len;
  const int64_t tk = k0 + (kok ? j : kv_len - 1);
  uint4 kf[KS], vf[KS];
  {
    const bf16_t* kp = p.k + tk * p.skt + (int64_t)kvh * p.skh;
    const bf16_t* vp = p.v + tk * p.svt + (int64_t)kvh * p.svh;
#pragma unroll
    for (int s = 0; s < KS; s++) {
      kf[s] = bwd_frag<PAD>(kp, s, dk_n, elem, true);
      vf[s] = bwd_frag<PAD>(vp, s, dv_n, elem, true);
    }
  }
  const float c2 = p.scale * 1.44269504f;
  f32x4 dk[NDS][8], dv[NDS][8];
#pragma unroll
  for (int ds = 0; ds < NDS; ds++)
#pragma unroll
    for (int td = 0; td < 8; td++) {
      dk[ds][td] = f32x4{0.f, 0.f, 0.f, 0.f};
      dv[ds][td] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  // The moving blocks of 64 queries start at the first query that sees the first key of the tile's 128-key group, as
  // in the LDS kernel (whose workgroup owns 128 keys): the same grouping of a key's queries into MFMA k-chunks,
  // hence the same bits in either kernel. Blocks whose queries all precede the tile contribute exact zeros.
  const int istart = max(0, (j0 & ~127) - shift);
  if (qlen > 0) {
    for (int hh = 0; hh < G; hh++) {
      const int h = kvh * G + hh;
      const bf16_t* qb_ = p.q + (int64_t)q0 * p.sqt + (int64_t)h * p.sqh;
      const bf16_t* db_ = p.d_o + (int64_t)q0 * p.sdt + (int64_t)h * p.sdh;
      for (int ib = istart; ib < qlen; ib += 64) {
        // phase 1: the block's Q and dO rows as A operands plus the rows' lse and delta (head sizes up to 128: all
        // loads first)
        uint4 qfr[HOIST ? 4 : 1][KS], ofr[HOIST ? 4 : 1][KS];
        float lse2[4][4], dl[4][4];
        auto load_tile = [&](int tt, int slot) {
          const int64_t ir = min(ib + 16 * tt + r16, qlen - 1);
#pragma unroll
          for (int s = 0; s < KS; s++) {
            qfr[slot][s] = bwd_frag<PAD>(qb_ + ir * p.sqt, s, dk_n, elem, false);
            ofr[slot][s] = bwd_frag<PAD>(db_ + ir * p.sdt, s, dv_n, elem, false);
          }
        };
#pragma unroll
        for (int tt = 0; tt < 4; tt++) {
          if constexpr (HOIST) load_tile(tt, tt);
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const int64_t tq = q0 + min(ib + 16 * tt + 4 * g + r, qlen - 1);
            lse2[tt][r] = p.lse[tq * p.Hq + h];
            dl[tt][r] = p.delta[tq * p.Hq + h];
          }
        }
        float pr[4][4], ds_[4][4];
#pragma unroll
        for (int tt = 0; tt < 4; tt++) {
          if constexpr (!HOIST) load_tile(tt, 0);
          const int slot = HOIST ? tt : 0;
          f32x4 st = f32x4{0.f, 0.f, 0.f, 0.f}, dp = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < KS; s++) {
            st = ET::mfma(qfr[slot][s], kf[s], st);
            dp = ET::mfma(ofr[slot][s], vf[s], dp);
          }
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const int iq = ib + 16 * tt + 4 * g + r;    // this register's query (moving row)
            const bool ok = iq < qlen && kok && j <= shift + iq;
            const float e = ok ? __builtin_amdgcn_exp2f(__builtin_fmaf(st[r], c2, -(lse2[tt][r] * 1.44269504f))) : 0.f;
            pr[tt][r] = e;
            ds_[tt][r] = e * (dp[r] - dl[tt][r]) * p.scale;
          }
        }
        // phase 2: the same rows in the transposable layout (they are in the cache now)
        uint4 pfp[2], pfs[2];
        bwd_pack<ET>(pr, pfp);
        bwd_pack<ET>(ds_, pfs);
#pragma unroll
        for (int ds = 0; ds < NDS; ds++) {
          uint4 rows_o[2][8], rows_q[2][8];
          bwd_tr_load<PAD>([&](int r) { return db_ + (int64_t)min(ib + r, qlen - 1) * p.sdt; }, ds, dv_n, elem, rows_o);
          bwd_tr_load<PAD>([&](int r) { return qb_ + (int64_t)min(ib + r, qlen - 1) * p.sqt; }, ds, dk_n, elem, rows_q);
          bwd_tr_product<ET>(rows_o, ds, dv_n, pfp, dv[ds]);
          bwd_tr_product<ET>(rows_q, ds, dk_n, pfs, dk[ds]);
        }
      }
    }
  }
  if (kok) {
#pragma unroll
    for (int ds = 0; ds < NDS; ds++) {
      bwd_store_tile<ET, PAD>(dk[ds], ds, dk_n, elem, p.dk + tk * p.sdkt + (int64_t)kvh * p.sdkh);
      bwd_store_tile<ET, PAD>(dv[ds], ds, dv_n, elem, p.dv + tk * p.sdvt + (int64_t)kvh * p.sdvh);
    }
  }
}

// delta, dQ, dK / dV with the register-form kernels
template <class ET, int D, bool PAD>
static int launch_attn_bwd_generic(const AttnBwdParams& p, int64_t total_q, int num_seqs, int max_q, int max_k, hipStream_t stream) {
  attn_bwd_delta_kernel<ET, D, PAD><<<(unsigned)((total_q * p.Hq + 15) / 16), 256, 0, stream>>>(p, total_q);
  attn_bwd_dq_kernel<ET, D, PAD><<<dim3((unsigned)((max_q + 63) / 64), (unsigned)p.Hq, (unsigned)num_seqs), 256, 0, stream>>>(p);
  attn_bwd_dkv_kernel<ET, D, PAD><<<dim3((unsigned)((max_k + 63) / 64), (unsigned)p.Hkv, (unsigned)num_seqs), 256, 0, stream>>>(p);
  return launch_status();
}

// fp16 (attn_bwd_f16.hip): Db = the built-for head size, 64, 128 or 256
int launch_attn_bwd_f16(const AttnBwdParams& p, int Db, int64_t total_q, int num_seqs, int max_q, int max_k, hipStream_t stream);

}  // namespace vx
