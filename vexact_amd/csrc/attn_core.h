// Causal GQA attention over a paged (or packed) KV cache for decode and chunked prefill, plus
// the KV-cache row scatter.
// Replaces _paged_attn_fwd_block_kernel / _PagedFlashAttentionVarlen
// (vexact/batch_invariant_ops/triton_invariant_attention.py:433-692), the forward of the packed
// twin _varlen_attn_fwd_block_kernel (:47-190, :700-784) and _store_cache_kernel / store_kvcache
// (vexact/batch_invariant_ops/kv_cache_context.py:259-314).
//
// Arithmetic per query row at absolute position p (keys 0..p visible), c = scale * log2(e):
//   keys are cut into chunks of 256 (absolute positions), each chunk into blocks of 64.
//   chunk state (m, l, acc) starts at (-inf, 0, 0); for each block, ascending:
//     t_i = fl(s_i * c), masked keys -> -inf ; m' = max(m, max_i t_i) ; a = exp2(m - m')
//     pb_i = r16(exp2(t_i - m')) ; acc = acc * a + sum_i pb_i * V_i (bf16 MFMA) ; l = l * a + sum_i pb_i
//   running state (M, L, ACC) folds the chunks in ascending order:
//     M' = max(M, m) ; A = exp2(M - M') ; B = exp2(m - M') ; L = L*A + l*B ; ACC = ACC*A + acc*B
//   out = r16(ACC / L)
// The decode kernel gives every (sequence, kv head, chunk) to one wavefront, writes the chunk
// states to a workspace and a second kernel folds them; the prefill kernel does the same fold in
// registers. Both run the same block routine, so a token's output has the same bits whether it
// is computed as the last row of a prefill chunk, as a decode step, alone or inside a batch.
//
// Layout trick: S is computed transposed (keys on MFMA rows, query rows on MFMA columns), so a
// lane's 4 results belong to one query row and softmax statistics stay in-lane; the bf16 P
// values are then already in MFMA B-operand order if the contraction slot (g, idx) of a 32-key
// chunk is mapped to key 16*(idx/4) + 4*g + idx%4. V rows are fetched in that key order with
// 16 lanes covering one 256-byte row, and an in-register 8x8 transpose turns 8 rows x 8 dims
// into 8 A-operand fragments, each feeding the MFMA for dims {8 i + t}.
#include "common.h"

#pragma once
namespace vx {

constexpr int ATT_CHUNK = 256;  // keys per split chunk (absolute positions)
constexpr int ATT_BLOCK = 64;   // keys per online-softmax block
constexpr float ATT_LAZY = 8.f; // log2 headroom before a row's reference maximum moves

struct AttnParams {
  const bf16_t* q;  // [T, Hq, DK]
  int64_t sqt, sqh;
  const bf16_t* k;  // paged: [blocks, page, Hkv, DK]; packed: [Tk, Hkv, DK]
  int64_t skb, skp, skh;  // packed: skp = row stride, skb unused
  const bf16_t* v;
  int64_t svb, svp, svh;
  bf16_t* o;  // [T, Hq, DV]
  int64_t sot, soh;
  const int* cu_q;       // [B+1]
  const int* seqused_k;  // paged: [B] kv lengths (clamped to max_kv: a wrong length must not walk off the block table)
  int max_kv;            // paged: keys a block-table row can address
  const int* cu_k;       // packed: [B+1]
  const int* block_table;  // [B, bt_stride]
  int64_t bt_stride;
  int page_size, page_shift;  // shift = -1 if not a power of two
  int Hq, Hkv, num_seqs;
  float qk_scale;  // scale * log2(e)
  int causal;
  // decode split workspace: one register image per (sequence, kv head, chunk), see part_image_floats
  float* part;
  int64_t img_floats;
  int max_chunks;
  const int* seq_order;  // optional [B]: decode kernels take sequence seq_order[i] as their i-th (longest first balances the tail)
  float* lse;  // optional [T, Hq]: natural-log sum of exp(scale * s) over a row's visible keys (general kernels)
  // General launches over batches whose sequences differ in their number of query rows:
  int compact;      // != 0: (sequence, row block) pairs are numbered compactly, see locate_row_block
  int grid_heads, grid_sg;  // plain form: head groups and sequences per group of sequences in blockIdx.x
  // Head sizes as the caller has them (the kernels' DK / DV template sizes are the next size they are built for; the
  // columns in between are fed to the matrix core as zeros and never stored); elem != 0: rows are not 16-byte
  // addressable (a head size or stride that is not a multiple of 8 elements), every access is per element.
  int dk, dv, elem;
  int single_mode;  // 0: every sequence; 1: only sequences with one query row (decode kernels inside a general
                    // launch); 2: all others (the general kernel beside them)
};

// Which sequence, which of its row blocks (rpb query rows each) and which group of heads a workgroup of a general
// kernel works on. Plain form: a grid of (head groups x grid_sg sequences) x ceil(max_q / rpb) x groups of sequences,
// most of it empty when one long chunk shares a batch with decode tokens. Workgroup ids go round the eight XCDs and
// are dispatched in order, so the fastest index holds what has equal work (the head groups of a few sequences, eight
// ids in all) and the row block comes next, running downwards: under a causal mask a sequence's blocks that see the
// most keys start first and its short ones fill the tail. (With the row block as the fastest index, a multiple of 8
// blocks per sequence pinned every block height to one XCD and long blocks started last.) Compact form: item w
// (see below for where it comes from) belongs to the last sequence s with cu_q[s] / rpb + s <= w, as its row block
// w - (cu_q[s] / rpb + s); every sequence owns at least ceil(qlen / rpb) items and there are total_q / rpb + num_seqs
// in all. Returns false when there is nothing to do.
__device__ __forceinline__ bool locate_row_block(const AttnParams& p, int rpb, int& seq, int& bx, int& hg) {
  if (!p.compact) {
    hg = (int)(blockIdx.x % p.grid_heads);
    bx = (int)(gridDim.y - 1 - blockIdx.y);
    seq = (int)(blockIdx.z * p.grid_sg + blockIdx.x / p.grid_heads);
    return seq < p.num_seqs;
  }
  // compact == 1: head group fastest, items downwards (a sequence's last row blocks, which see the most keys, first);
  // compact == 2 (more items than blockIdx.y can count): items in blockIdx.x, upwards
  hg = p.compact == 1 ? blockIdx.x : blockIdx.y;
  const int w = p.compact == 1 ? (int)(gridDim.y - 1 - blockIdx.y) : (int)blockIdx.x;
  int lo = 0, hi = p.num_seqs - 1;
  while (lo < hi) {  // cu_q[s] / rpb + s is strictly increasing in s
    const int mid = (lo + hi + 1) >> 1;
    if (p.cu_q[mid] / rpb + mid <= w) lo = mid;
    else hi = mid - 1;
  }
  seq = lo;
  bx = w - (p.cu_q[lo] / rpb + lo);
  return bx >= 0;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// sequence handled by decode workgroup i (clamped: a bad order entry must not become a wild address)
__device__ __forceinline__ int decode_seq(const AttnParams& p, unsigned i) {
  return p.seq_order ? min(max(p.seq_order[i], 0), p.num_seqs - 1) : (int)i;
}

// Where a sequence's keys and values live. SRC_FAST: paged, page size a power of two >= 16, so a
// 16-key tile lies inside one page and its page id is wave-uniform. SRC_GENERIC: paged, any page
// size (one table lookup per key). SRC_PACKED: contiguous rows [Tk, Hkv, D].
enum : int { SRC_FAST = 0, SRC_GENERIC = 1, SRC_PACKED = 2 };

template <int KIND>
struct KVSource {
  const bf16_t* kbase;  // + kv head offset (packed: + first key of the sequence)
  const bf16_t* vbase;
  const int* bt;        // this sequence's block-table row
  int64_t skb, skp, svb, svp;
  int ps, shift, last;  // last = kv_len - 1; every address is clamped to an existing key

  struct Tiles { int pg[4], off[4]; };  // page id and first in-page row of the four 16-key tiles of a block

  __device__ __forceinline__ Tiles tiles(int kb) const {
    Tiles t;
#pragma unroll
    for (int tt = 0; tt < 4; tt++) {
      t.pg[tt] = 0; t.off[tt] = 0;
      if constexpr (KIND == SRC_FAST) {
        const int key = kb + 16 * tt;
        const int kk = key <= last ? key : 0;  // a tile past the end is never dereferenced for real
        t.pg[tt] = bt[kk >> shift];
        t.off[tt] = kk & (ps - 1);
      }
    }
    return t;
  }
  // row of key kb + 16 tt + within; `within` must already be 0 for keys past the end (FAST)
  __device__ __forceinline__ const bf16_t* krow(const Tiles& t, int kb, int tt, int within) const {
    if constexpr (KIND == SRC_FAST) return kbase + (int64_t)t.pg[tt] * skb + (int64_t)(t.off[tt] + within) * skp;
    const int key = min(kb + 16 * tt + within, last);
    if constexpr (KIND == SRC_PACKED) return kbase + (int64_t)key * skp;
    int pg, off;
    if (shift >= 0) { pg = key >> shift; off = key & (ps - 1); }
    else { pg = key / ps; off = key - pg * ps; }
    return kbase + (int64_t)bt[pg] * skb + (int64_t)off * skp;
  }
  __device__ __forceinline__ const bf16_t* vrow(const Tiles& t, int kb, int tt, int within) const {
    if constexpr (KIND == SRC_FAST) return vbase + (int64_t)t.pg[tt] * svb + (int64_t)(t.off[tt] + within) * svp;
    const int key = min(kb + 16 * tt + within, last);
    if constexpr (KIND == SRC_PACKED) return vbase + (int64_t)key * svp;
    int pg, off;
    if (shift >= 0) { pg = key >> shift; off = key & (ps - 1); }
    else { pg = key / ps; off = key - pg * ps; }
    return vbase + (int64_t)bt[pg] * svb + (int64_t)off * svp;
  }
};

// Online-softmax update of one 16-query tile from the raw score tiles st (S^T: lane holds keys
// kb + 16 tt + 4 g + r of query column r16) of the 64-key block at kb: masks keys past qpos, updates
// the running max m and sum l, rescales the NACC accumulators and packs P (rounded to bf16; the sum
// uses the rounded values) as the two B operands of the P V MFMAs. Shared by every attention kernel.
// op(x, x of lane ^ 16) and op(x, x of lane ^ 32) for a commutative op, through the row-swap instructions
// (v_permlane16_swap / v_permlane32_swap: the odd 16-lane rows of the first register trade places with the
// even rows of the second, resp. rows 2, 3 with rows 0, 1). With both registers holding x, the two results
// hold the lane's own row pair member and its partner's: no LDS round trip as with a general shuffle.
// Written as asm: through the builtins the compiler used the first result for both (seen in the generated
// code of this toolchain). The s_nop covers the wait states between a vector write of an operand and the swap.
__device__ __forceinline__ void swap16(float x, float& a, float& b) {
  a = x; b = x;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap32(float x, float& a, float& b) {
  a = x; b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float max_xor16(float x) { float a, b; swap16(x, a, b); return fmaxf(a, b); }
__device__ __forceinline__ float max_xor32(float x) { float a, b; swap32(x, a, b); return fmaxf(a, b); }
__device__ __forceinline__ float add_xor16(float x) { float a, b; swap16(x, a, b); return a + b; }
__device__ __forceinline__ float add_xor32(float x) { float a, b; swap32(x, a, b); return a + b; }

template <class ET, int NACC>
__device__ __forceinline__ void attn_softmax_tile(f32x4 (&st)[4], int kb, float c, int qpos, float& m, float& l,
                                                  f32x4 (&acc)[NACC], uint4 (&pf)[2], bool all_visible = false) {
  const int lane = threadIdx.x & 63, g = lane >> 4;
  // The block maximum is taken over the raw scores and scaled once: x -> fl(x c) is monotone for
  // c > 0, so fl(max(s) c) = max(fl(s c)); the exponent argument is then one fused multiply-add.
  float bm = -INFINITY;
  if (all_visible) {  // wave-uniform: every key of the block is visible to every row of the tile
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
#pragma unroll
      for (int r = 0; r < 4; r++) bm = fmaxf(bm, st[tt][r]);
  } else {
    // key kb + 16 tt + 4 g + r is visible iff 16 tt + r <= lim: the comparisons then have constant left sides
    const int lim = qpos - kb - 4 * g;
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const float tv = (16 * tt + r <= lim) ? st[tt][r] : -INFINITY;  // exp2(fma(-inf, c, .)) = 0 below
        st[tt][r] = tv;
        bm = fmaxf(bm, tv);
      }
  }
  bm = max_xor16(bm);
  bm = max_xor32(bm);
  bm = bm * c;
  // m is the reference point of the row's exponents, not necessarily its maximum: it moves only when the
  // block's maximum exceeds it by more than ATT_LAZY (then probabilities stay below 2^ATT_LAZY, harmless
  // in bf16 / fp32), so most blocks leave the accumulators unscaled. A function of the row's own scores
  // only, hence the same in every kernel and for every batch.
  const float mn = (bm > m + ATT_LAZY) ? bm : m;
  const float ms = (mn == -INFINITY) ? 0.f : mn;  // fully masked so far: everything stays 0
  const float alpha = fast_exp2(m - ms);
  float rs = 0.f;
  uint32_t pw[4][2];
#pragma unroll
  for (int tt = 0; tt < 4; tt++) {
#pragma unroll
    for (int h = 0; h < 2; h++) {
      // two probabilities rounded to bf16 at once; the row sum adds the rounded values (one
      // v_dot2c_f32_bf16 with a pair of ones adds both halves)
      const uint32_t pk = ET::pack2(fast_exp2(__builtin_fmaf(st[tt][2 * h], c, -ms)),
                                    fast_exp2(__builtin_fmaf(st[tt][2 * h + 1], c, -ms)));
      rs = ET::add2(pk, rs);
      pw[tt][h] = pk;
    }
  }
  rs = add_xor16(rs);
  rs = add_xor32(rs);
  l = l * alpha + rs;
  const bool had_keys = m != -INFINITY;
  m = mn;
  // multiplying by exactly 1 changes nothing, and a row that had seen no key holds exact zeros: skip the
  // rescale unless some lane's reference moved away from a finite value
  if (__builtin_amdgcn_ballot_w64(alpha != 1.0f && had_keys) != 0) {
#pragma unroll
    for (int i = 0; i < NACC; i++) {
      acc[i][0] *= alpha; acc[i][1] *= alpha; acc[i][2] *= alpha; acc[i][3] *= alpha;
    }
  }
  pf[0] = make_uint4(pw[0][0], pw[0][1], pw[1][0], pw[1][1]);
  pf[1] = make_uint4(pw[2][0], pw[2][1], pw[3][0], pw[3][1]);
}

// Eight consecutive elements of a row starting at column col, of a row that has d valid columns. Exact head sizes
// (PAD = false): one 16-byte load. Padded head sizes: a piece that starts at or past d re-reads the row's first piece
// (a dereferenceable address; what it returns meets a zero on the other side of its product, or lands in output columns
// that are never stored); with elem set the row is not 16-byte addressable and the piece is gathered element by
// element, zeros past d.
template <bool PAD>
__device__ __forceinline__ uint4 attn_ld8(const bf16_t* row, int col, int d, int elem) {
  if constexpr (!PAD) {
    return ldg16_raw(row + col);
  } else {
    if (!elem) return ldg16_raw(row + (col < d ? col : 0));
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int c0 = col + 2 * i, c1 = c0 + 1;
      const uint32_t lo = row[min(c0, d - 1)], hi = row[min(c1, d - 1)];
      w[i] = (c0 < d ? lo : 0u) | ((c1 < d ? hi : 0u) << 16);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
  }
}
// Eight consecutive output elements (packed pairs in pk) to columns d0 .. d0 + 7 of a row with dv columns.
template <bool PAD>
__device__ __forceinline__ void attn_st8(bf16_t* row, int d0, uint4 pk, int dv, int elem) {
  if constexpr (!PAD) {
    *(uint4*)(row + d0) = pk;
  } else {
    if (!elem) {
      if (d0 < dv) *(uint4*)(row + d0) = pk;
      return;
    }
    const uint32_t w[4] = {pk.x, pk.y, pk.z, pk.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if (d0 + 2 * i < dv) row[d0 + 2 * i] = (bf16_t)(w[i] & 0xffffu);
      if (d0 + 2 * i + 1 < dv) row[d0 + 2 * i + 1] = (bf16_t)(w[i] >> 16);
    }
  }
}
// The same for four elements (dv is a multiple of 4 whenever elem is 0 on a padded size)
template <bool PAD>
__device__ __forceinline__ void attn_st4(bf16_t* row, int d0, uint2 pk, int dv, int elem) {
  if constexpr (!PAD) {
    *(uint2*)(row + d0) = pk;
  } else {
    if (!elem) {
      if (d0 < dv) *(uint2*)(row + d0) = pk;
      return;
    }
    const uint32_t w[2] = {pk.x, pk.y};
#pragma unroll
    for (int i = 0; i < 2; i++) {
      if (d0 + 2 * i < dv) row[d0 + 2 * i] = (bf16_t)(w[i] & 0xffffu);
      if (d0 + 2 * i + 1 < dv) row[d0 + 2 * i + 1] = (bf16_t)(w[i] >> 16);
    }
  }
}

// ET: element type (ElemBF16 / ElemF16); DK, DV: head sizes the code is built for; PAD: the caller's head sizes
// (dk <= DK, dv <= DV) may be smaller. Columns dk .. DK of the queries are zeros, so whatever the key loads return
// there adds exact zeros to the end of each score's ascending chain: the scores, and with them every output bit, are
// those of an exact-size kernel. Output columns dv .. DV are computed from re-read data and dropped.
template <class ET, int DK, int DV, int QT, bool PAD>
struct AttnWave {
  static constexpr int KS = DK / 32;           // MFMA k-steps for S
  static constexpr int NDV = (DV + 127) / 128;  // sets of 8 PV MFMAs
  static constexpr int NACC = NDV * 8;

  // per q-tile, per lane (column j = lane % 16)
  uint4 qf[QT][KS];
  int qpos[QT];  // last visible key of this lane's query row; -1 = row not valid
  float m[QT], l[QT];
  f32x4 acc[QT][NACC];
  // K and V of the block being worked on / in flight
  uint4 kf[4][KS];
  uint4 vr[2][NDV][8];  // [32-key chunk][dim set][slot]
  int dk, dv, elem;     // the caller's head sizes (PAD only; otherwise DK, DV, 0)

  __device__ __forceinline__ void init_sizes(const AttnParams& p) {
    if constexpr (PAD) { dk = p.dk; dv = p.dv; elem = p.elem; }
    else { dk = DK; dv = DV; elem = 0; }
  }

  // query row fragment for tile t: dims 32 s + 8 g .. +8 of the row at qrow, zeros if the row is not valid or the
  // dims lie past dk
  __device__ __forceinline__ void load_q(int t, const bf16_t* qrow, bool ok) {
    const int g = (threadIdx.x & 63) >> 4;
#pragma unroll
    for (int s = 0; s < KS; s++) {
      const int col = 32 * s + 8 * g;
      qf[t][s] = mask16(attn_ld8<PAD>(qrow, col, dk, elem), ok && (!PAD || col < dk));
    }
  }

  __device__ __forceinline__ void reset_chunk() {
#pragma unroll
    for (int t = 0; t < QT; t++) {
      m[t] = -INFINITY;
      l[t] = 0.f;
#pragma unroll
      for (int i = 0; i < NACC; i++) acc[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }

  // lane (r16, g) fetches key 16 tt + r16, dims 32 s + 8 g .. +8: the MFMA A operand of S^T.
  // Keys past the end read an existing row instead; their scores are set to -inf later.
  template <typename Src>
  __device__ __forceinline__ void issue_k(const Src& src, const typename Src::Tiles& tl, int kb, int kv_len) {
    const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
#pragma unroll
    for (int tt = 0; tt < 4; tt++) {
      const bool ok = kb + 16 * tt + r16 < kv_len;
      const bf16_t* kp = src.krow(tl, kb, tt, ok ? r16 : 0);
#pragma unroll
      for (int s = 0; s < KS; s++) kf[tt][s] = attn_ld8<PAD>(kp, 32 * s + 8 * g, dk, elem);
    }
  }
  // lane (r16, g) fetches, for slot idx of 32-key chunk ch, key 32 ch + 16 (idx/4) + 4 g + idx%4,
  // dims 8 r16 .. +8 (16 lanes cover one 256-byte row)
  template <typename Src>
  __device__ __forceinline__ void issue_v(const Src& src, const typename Src::Tiles& tl, int kb, int kv_len) {
    const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
#pragma unroll
    for (int ch = 0; ch < 2; ch++)
#pragma unroll
      for (int idx = 0; idx < 8; idx++) {
        const int tt = 2 * ch + (idx >> 2), within = 4 * g + (idx & 3);
        const bool ok = kb + 16 * tt + within < kv_len;
        const bf16_t* vp = src.vrow(tl, kb, tt, ok ? within : 0);
#pragma unroll
        for (int ds = 0; ds < NDV; ds++) {
          if constexpr (PAD) {
            vr[ch][ds][idx] = attn_ld8<true>(vp, 128 * ds + 8 * r16, dv, elem);
          } else {
            const bool dok = 128 * ds + 8 * r16 < DV;
            vr[ch][ds][idx] = ldg16_raw(vp + (dok ? 128 * ds + 8 * r16 : 0));
          }
        }
      }
  }

  // scores of the 64-key block at kb from kf, online-softmax update, P packed for the PV MFMAs
  __device__ __forceinline__ void scores(int kb, float c, uint4 (&pf)[QT][2]) {
#pragma unroll
    for (int t = 0; t < QT; t++) {
      // S^T tiles: lane holds keys kb + 16 tt + 4 g + r for query column r16
      f32x4 st[4];
#pragma unroll
      for (int tt = 0; tt < 4; tt++) {
        st[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; s++) st[tt] = ET::mfma(kf[tt][s], qf[t][s], st[tt]);
      }
      softmax_tile(t, st, kb, c, pf);
    }
  }

  // online-softmax update of q-tile t from the raw score tiles st of the 64-key block at kb
  __device__ __forceinline__ void softmax_tile(int t, f32x4 (&st)[4], int kb, float c, uint4 (&pf)[QT][2]) {
    attn_softmax_tile<ET>(st, kb, c, qpos[t], m[t], l[t], acc[t], pf[t]);
  }

  // acc += P V with the block's values in vr. Values of keys past the end are zeroed first (their
  // probability is 0, but 0 * garbage could be NaN).
  __device__ __forceinline__ void pv(int kb, int kv_len, const uint4 (&pf)[QT][2]) {
    const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
    const bool tail = kb + ATT_BLOCK > kv_len;  // wave-uniform: only a sequence's last block
#pragma unroll
    for (int ch = 0; ch < 2; ch++)
#pragma unroll
      for (int ds = 0; ds < NDV; ds++) {
        uint4 row[8];
#pragma unroll
        for (int idx = 0; idx < 8; idx++) {
          row[idx] = vr[ch][ds][idx];
          // built-for sizes below 128: the lanes past DV hold re-read data and are zeroed; padded sizes leave such
          // lanes alone (their output columns are never stored)
          const bool dok = PAD || 128 * ds + 8 * r16 < DV;
          if (tail || !dok) {
            const bool ok = kb + 16 * (2 * ch + (idx >> 2)) + 4 * g + (idx & 3) < kv_len;
            row[idx] = mask16(row[idx], ok && dok);
          }
        }
#pragma unroll
        for (int td = 0; td < 8; td++) {
          // 8x8 transpose of 16-bit elements: fragment td takes dim 8 r16 + td of the 8 key slots
          uint32_t w[4];
#pragma unroll
          for (int qd = 0; qd < 4; qd++) {
            const uint4 ra = row[2 * qd], rb = row[2 * qd + 1];
            const uint32_t a = (td < 2) ? ra.x : (td < 4) ? ra.y : (td < 6) ? ra.z : ra.w;
            const uint32_t b = (td < 2) ? rb.x : (td < 4) ? rb.y : (td < 6) ? rb.z : rb.w;
            w[qd] = (td & 1) ? ((a >> 16) | (b & 0xffff0000u)) : ((a & 0xffffu) | (b << 16));
          }
          const uint4 vf = make_uint4(w[0], w[1], w[2], w[3]);
#pragma unroll
          for (int t = 0; t < QT; t++) acc[t][ds * 8 + td] = ET::mfma(vf, pf[t][ch], acc[t][ds * 8 + td]);
        }
      }
  }

  // One chunk: keys [kb0, kb_end) in 64-key blocks, chunk state reset first. The loads of block
  // b+1 are issued as soon as block b has consumed the registers they land in (K after the score
  // MFMAs, V after the PV MFMAs), so a wavefront always has a block of K or V in flight.
  template <typename Src>
  __device__ __forceinline__ void run_chunk(const Src& src, int kb0, int kb_end, int kv_len, float c) {
    reset_chunk();
    typename Src::Tiles tl = src.tiles(kb0);
    issue_k(src, tl, kb0, kv_len);
    issue_v(src, tl, kb0, kv_len);
    for (int kb = kb0; kb < kb_end; kb += ATT_BLOCK) {
      const bool more = kb + ATT_BLOCK < kb_end;
      if (more) tl = src.tiles(kb + ATT_BLOCK);  // page ids of the next block: ready before they are needed
      uint4 pf[QT][2];
      scores(kb, c, pf);
      if (more) issue_k(src, tl, kb + ATT_BLOCK, kv_len);
      pv(kb, kv_len, pf);
      if (more) issue_v(src, tl, kb + ATT_BLOCK, kv_len);
    }
  }
};

// running = running * A + chunk * B, the same expression (one product, one fused multiply-add) wherever chunk
// states are folded, so that every kernel gives the same bits
__device__ __forceinline__ float fold_add(float running, float A, float chunk, float B) {
  return __builtin_fmaf(running, A, chunk * B);
}

// fold a chunk state into the running state; exact no-op for an all-masked chunk
__device__ __forceinline__ void fold_scales(float M, float mc, float& Mn, float& A, float& B) {
  Mn = fmaxf(M, mc);
  const float ms = (Mn == -INFINITY) ? 0.f : Mn;
  A = fast_exp2(M - ms);
  B = fast_exp2(mc - ms);
}

template <int KIND>
__device__ __forceinline__ KVSource<KIND> make_source(const AttnParams& p, int seq, int kvh, int k0, int kv_len) {
  KVSource<KIND> s;
  s.skb = p.skb; s.skp = p.skp; s.svb = p.svb; s.svp = p.svp;
  s.ps = p.page_size; s.shift = p.page_shift; s.last = kv_len - 1;
  if constexpr (KIND == SRC_PACKED) {
    s.kbase = p.k + (int64_t)k0 * p.skp + (int64_t)kvh * p.skh;
    s.vbase = p.v + (int64_t)k0 * p.svp + (int64_t)kvh * p.svh;
    s.bt = nullptr;
  } else {
    s.kbase = p.k + (int64_t)kvh * p.skh;
    s.vbase = p.v + (int64_t)kvh * p.svh;
    s.bt = p.block_table + (int64_t)seq * p.bt_stride;
  }
  return s;
}

// ---------------------------------------------------------------------------------------
// Decode: every sequence has at most one query token. grid = (Hkv, B, max_chunks), one
// wavefront per block; query heads of the kv head are the MFMA columns (G <= 16 * QT).
// ---------------------------------------------------------------------------------------
template <class ET, int DK, int DV, int QT, int KIND, bool PAD>
__device__ __forceinline__ void attn_decode_split_body(const AttnParams& p) {
  const int kvh = blockIdx.x, seq = decode_seq(p, blockIdx.y), chunk = blockIdx.z;  // chunk slowest: late chunks, mostly empty, are dispatched last
  const int q0 = p.cu_q[seq];
  const int qlen = p.cu_q[seq + 1] - q0;
  const int kv_len = min(p.seqused_k[seq], p.max_kv);
  if (qlen <= 0 || kv_len <= 0) return;
  const int kstart = chunk * ATT_CHUNK;
  if (kstart >= kv_len) return;
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int G = p.Hq / p.Hkv;
  const int64_t tok = q0 + qlen - 1;  // the (only) query token
  const int pos = p.causal ? kv_len - 1 : kv_len - 1;

  AttnWave<ET, DK, DV, QT, PAD> w;
  w.init_sizes(p);
#pragma unroll
  for (int t = 0; t < QT; t++) {
    const int hl = 16 * t + r16;  // head within the group
    const bool ok = hl < G;
    w.qpos[t] = ok ? pos : -1;
    w.load_q(t, p.q + tok * p.sqt + (int64_t)(kvh * G + (ok ? hl : 0)) * p.sqh, ok);
  }
  const KVSource<KIND> src = make_source<KIND>(p, seq, kvh, 0, kv_len);
  w.run_chunk(src, kstart, min(kstart + ATT_CHUNK, kv_len), kv_len, p.qk_scale);

  // Write the chunk state as the wavefront holds it: float4 slot i of lane l lands at
  // image[(i * 64 + l) * 4], so every store instruction writes whole 128-byte lines (a layout by
  // head and dim would scatter 16-byte pieces). Slot ((t NDV + ds) 4 + r) 2 + h holds dims
  // 128 ds + 32 g + 8 r + 4 h .. +4 of head 16 t + r16; slot NI + t holds (m, l) of that head.
  constexpr int NDV = (DV + 127) / 128, NI = QT * NDV * 8;
  float4* ip = (float4*)(p.part + ((int64_t)(seq * p.Hkv + kvh) * p.max_chunks + chunk) * p.img_floats) + lane;
#pragma unroll
  for (int t = 0; t < QT; t++) {
    if (16 * t + r16 >= G) continue;
#pragma unroll
    for (int ds = 0; ds < NDV; ds++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        if (128 * ds + 32 * g + 8 * r >= w.dv) continue;
        const int sl = ((t * NDV + ds) * 4 + r) * 2;
        ip[sl * 64] = make_float4(w.acc[t][ds * 8 + 0][r], w.acc[t][ds * 8 + 1][r], w.acc[t][ds * 8 + 2][r],
                                  w.acc[t][ds * 8 + 3][r]);
        ip[(sl + 1) * 64] = make_float4(w.acc[t][ds * 8 + 4][r], w.acc[t][ds * 8 + 5][r],
                                        w.acc[t][ds * 8 + 6][r], w.acc[t][ds * 8 + 7][r]);
      }
    ip[(NI + t) * 64] = make_float4(w.m[t], w.l[t], 0.f, 0.f);
  }
}

// Two wavefronts per SIMD hide one wavefront's set-up and tail behind another's streaming; that
// needs <= 256 registers, which the one-q-tile variants up to head size 128 meet without spilling.
// The larger variants keep the full register file (one wavefront per SIMD).
template <class ET, int DK, int DV, int QT, int KIND, bool PAD>
__global__ __launch_bounds__(64) void attn_decode_split_kernel(AttnParams p) {
  attn_decode_split_body<ET, DK, DV, QT, KIND, PAD>(p);
}
template <class ET, int DK, int DV, int QT, int KIND, bool PAD>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2))) void attn_decode_split_kernel_occ2(AttnParams p) {
  attn_decode_split_body<ET, DK, DV, QT, KIND, PAD>(p);
}

// ---------------------------------------------------------------------------------------
// Decode, chunks folded inside the workgroup: grid = (Hkv, B), NW wavefronts per block. Wavefront v
// takes chunks v, v + NW, ... of its (sequence, kv head); after each round the NW chunk states go to
// LDS (same register image as the split kernel writes to HBM) and are folded, in ascending chunk
// order, into a running state that lives in LDS, one owner thread per (head, 4 dims). Same fold
// arithmetic as attn_decode_combine_kernel, so both decode paths give the same bits; this one has
// no HBM round trip for the chunk states and no second launch, but needs B * Hkv * NW wavefronts to
// fill the machine.
// ---------------------------------------------------------------------------------------
template <class ET, int DK, int DV, int QT, int KIND, int NW, bool PAD>
__device__ __forceinline__ void attn_decode_fused_body(const AttnParams& p) {
  constexpr int NDV = (DV + 127) / 128, NI = QT * NDV * 8;
  constexpr int IMG4 = (NI + QT) * 64;   // float4 per chunk image
  constexpr int MAXE = 16 * QT * (DV / 4);  // owner elements: (head, 4 dims)
  extern __shared__ __attribute__((aligned(16))) uint8_t fz_lds[];
  float4* img = (float4*)fz_lds;                    // [NW][IMG4]
  float4* racc = img + NW * IMG4;                   // [MAXE] running accumulators
  float2* rml = (float2*)(racc + MAXE);             // [MAXE] running (M, L), one private copy per element

  const int kvh = blockIdx.x, seq = decode_seq(p, blockIdx.y);
  const int q0 = p.cu_q[seq];
  const int qlen = p.cu_q[seq + 1] - q0;
  const int kv_len = min(p.seqused_k[seq], p.max_kv);
  if (qlen <= 0 || kv_len <= 0) return;  // uniform over the block
  if (p.single_mode == 1 && qlen != 1) return;  // inside a general launch: the general kernel takes these
  const int tid = threadIdx.x, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
  const int wave = tid >> 6;
  const int G = p.Hq / p.Hkv;
  const int64_t tok = q0 + qlen - 1;
  const int pos = kv_len - 1;
  const int nch = (kv_len + ATT_CHUNK - 1) / ATT_CHUNK;
  const int nelem = G * (DV / 4);

  for (int e = tid; e < nelem; e += 64 * NW) {
    racc[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    rml[e] = make_float2(-INFINITY, 0.f);
  }

  AttnWave<ET, DK, DV, QT, PAD> w;
  w.init_sizes(p);
#pragma unroll
  for (int t = 0; t < QT; t++) {
    const int hl = 16 * t + r16;
    const bool ok = hl < G;
    w.qpos[t] = ok ? pos : -1;
    w.load_q(t, p.q + tok * p.sqt + (int64_t)(kvh * G + (ok ? hl : 0)) * p.sqh, ok);
  }
  const KVSource<KIND> src = make_source<KIND>(p, seq, kvh, 0, kv_len);

  for (int c0 = 0; c0 < nch; c0 += NW) {
    const int c = c0 + wave;
    if (c < nch) w.run_chunk(src, c * ATT_CHUNK, min(c * ATT_CHUNK + ATT_CHUNK, kv_len), kv_len, p.qk_scale);
    __syncthreads();  // the previous round's fold has finished reading the images
    if (c < nch) {
      float4* ip = img + wave * IMG4 + lane;
#pragma unroll
      for (int t = 0; t < QT; t++) {
        if (16 * t + r16 >= G) continue;
#pragma unroll
        for (int ds = 0; ds < NDV; ds++)
#pragma unroll
          for (int r = 0; r < 4; r++) {
            if (128 * ds + 32 * g + 8 * r >= w.dv) continue;
            const int sl = ((t * NDV + ds) * 4 + r) * 2;
            ip[sl * 64] = make_float4(w.acc[t][ds * 8 + 0][r], w.acc[t][ds * 8 + 1][r],
                                      w.acc[t][ds * 8 + 2][r], w.acc[t][ds * 8 + 3][r]);
            ip[(sl + 1) * 64] = make_float4(w.acc[t][ds * 8 + 4][r], w.acc[t][ds * 8 + 5][r],
                                            w.acc[t][ds * 8 + 6][r], w.acc[t][ds * 8 + 7][r]);
          }
        ip[(NI + t) * 64] = make_float4(w.m[t], w.l[t], 0.f, 0.f);
      }
    }
    __syncthreads();
    const int nr = min(NW, nch - c0);  // chunk states of this round
    for (int e = tid; e < nelem; e += 64 * NW) {
      const int hl = e / (DV / 4), d = 4 * (e % (DV / 4));
      const int t = hl >> 4, hr = hl & 15;
      const int sl = ((t * NDV + d / 128) * 4 + (d % 32) / 8) * 2 + (d % 8) / 4;
      const int ln = 16 * ((d % 128) / 32) + hr;
      float4 A4 = racc[e];
      float M = rml[e].x, L = rml[e].y;
      for (int j = 0; j < nr; j++) {
        const float4 ml = img[j * IMG4 + (NI + t) * 64 + hr];
        const float4 a = img[j * IMG4 + sl * 64 + ln];
        float Mn, A, B;
        fold_scales(M, ml.x, Mn, A, B);
        L = fold_add(L, A, ml.y, B);
        A4.x = fold_add(A4.x, A, a.x, B);
        A4.y = fold_add(A4.y, A, a.y, B);
        A4.z = fold_add(A4.z, A, a.z, B);
        A4.w = fold_add(A4.w, A, a.w, B);
        M = Mn;
      }
      racc[e] = A4;
      rml[e] = make_float2(M, L);
    }
  }
  // every thread reads back only what it wrote itself
  for (int e = tid; e < nelem; e += 64 * NW) {
    const int hl = e / (DV / 4), d = 4 * (e % (DV / 4));
    const float4 a = racc[e];
    const float L = rml[e].y;
    uint2 pk;
    pk.x = ET::pack2(a.x / L, a.y / L);
    pk.y = ET::pack2(a.z / L, a.w / L);
    attn_st4<PAD>(p.o + tok * p.sot + (int64_t)(kvh * G + hl) * p.soh, d, pk, w.dv, w.elem);
  }
}

template <class ET, int DK, int DV, int QT, int KIND, int NW, bool PAD>
__global__ __launch_bounds__(64 * NW) void attn_decode_fused_kernel(AttnParams p) {
  attn_decode_fused_body<ET, DK, DV, QT, KIND, NW, PAD>(p);
}
template <class ET, int DK, int DV, int QT, int KIND, int NW, bool PAD>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2))) void attn_decode_fused_kernel_occ2(AttnParams p) {
  attn_decode_fused_body<ET, DK, DV, QT, KIND, NW, PAD>(p);
}

template <int DV, int QT, int NW>
constexpr int fused_lds_bytes() {
  return (NW * (QT * ((DV + 127) / 128) * 8 + QT) * 64 + 16 * QT * (DV / 4)) * 16 + 16 * QT * (DV / 4) * 8;
}

// Folds the chunk images of one (sequence, kv head) in ascending chunk order. grid = (Hkv, B),
// one wavefront with the lane layout of the split kernel: lane (r16, g) owns head 16 t + r16, dims
// 128 ds + 32 g + 8 r + (0..7), reads its own slots of every image and writes 16 bytes per (ds, r).
template <class ET, int DV, int QT, bool PAD>
__global__ __launch_bounds__(64) void attn_decode_combine_kernel(AttnParams p) {
  const int dv = PAD ? p.dv : DV, elem = PAD ? p.elem : 0;
  const int kvh = blockIdx.x, seq = decode_seq(p, blockIdx.y);
  const int q0 = p.cu_q[seq];
  const int qlen = p.cu_q[seq + 1] - q0;
  const int kv_len = min(p.seqused_k[seq], p.max_kv);
  if (qlen <= 0 || kv_len <= 0) return;
  const int nch = (kv_len + ATT_CHUNK - 1) / ATT_CHUNK;
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int G = p.Hq / p.Hkv;
  constexpr int NDV = (DV + 127) / 128, NI = QT * NDV * 8;
  const float4* ip0 = (const float4*)(p.part + (int64_t)(seq * p.Hkv + kvh) * p.max_chunks * p.img_floats) + lane;
  const int64_t tok = q0 + qlen - 1;
#pragma unroll
  for (int t = 0; t < QT; t++) {
    const int hl = 16 * t + r16;
    if (hl >= G) continue;
    float M = -INFINITY, L = 0.f;
    float4 ACC[NDV * 8];
#pragma unroll
    for (int i = 0; i < NDV * 8; i++) ACC[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int c = 0; c < nch; c++) {
      const float4* ip = ip0 + (int64_t)c * (p.img_floats / 4);
      const float4 ml = ip[(NI + t) * 64];
      float Mn, A, B;
      fold_scales(M, ml.x, Mn, A, B);
      L = fold_add(L, A, ml.y, B);
#pragma unroll
      for (int i = 0; i < NDV * 8; i++) {
        const int ds = i >> 3, r = (i >> 1) & 3;
        if (128 * ds + 32 * g + 8 * r >= dv) continue;
        const float4 a = ip[(t * NDV * 8 + i) * 64];
        ACC[i].x = fold_add(ACC[i].x, A, a.x, B);
        ACC[i].y = fold_add(ACC[i].y, A, a.y, B);
        ACC[i].z = fold_add(ACC[i].z, A, a.z, B);
        ACC[i].w = fold_add(ACC[i].w, A, a.w, B);
      }
      M = Mn;
    }
    bf16_t* op = p.o + tok * p.sot + (int64_t)(kvh * G + hl) * p.soh;
#pragma unroll
    for (int ds = 0; ds < NDV; ds++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int d0 = 128 * ds + 32 * g + 8 * r;
        if (d0 >= dv) continue;
        const float4 lo = ACC[(ds * 4 + r) * 2], hi = ACC[(ds * 4 + r) * 2 + 1];
        uint4 pk;
        pk.x = ET::pack2(lo.x / L, lo.y / L);
        pk.y = ET::pack2(lo.z / L, lo.w / L);
        pk.z = ET::pack2(hi.x / L, hi.y / L);
        pk.w = ET::pack2(hi.z / L, hi.w / L);
        attn_st8<PAD>(op, d0, pk, dv, elem);
      }
  }
}

// ---------------------------------------------------------------------------------------
// General (prefill / mixed / packed) kernel. grid = (q tiles, Hq, B); 4 wavefronts per block,
// wavefront v owns query rows [64 QT bx + 16 QT v, +16 QT) of the sequence (local indices).
// ---------------------------------------------------------------------------------------
template <class ET, int DK, int DV, int QT, int KIND, bool PAD>
__global__ __launch_bounds__(256) void attn_prefill_kernel(AttnParams p, int hpw) {
  // The 4 * QT query tiles (16 rows each) of a block are spread over hpw query heads of one kv head
  // and 4 * QT / hpw row tiles: tile slot s = wave * QT + t -> head s % hpw, row tile s / hpw. With
  // hpw > 1 the wavefronts of a block walk the same keys at the same time, so K and V mostly come
  // from the CU's L1 after the first wavefront has fetched them.
  const int rows_per_block = 16 * (4 * QT / hpw);
  int seq, bx, hg;
  if (!locate_row_block(p, rows_per_block, seq, bx, hg)) return;
  const int q0 = p.cu_q[seq];
  const int qlen = p.cu_q[seq + 1] - q0;
  if (p.single_mode == 2 && qlen == 1) return;  // a decode kernel of the same launch takes these
  int kv_len, k0 = 0;
  if constexpr (KIND != SRC_PACKED) kv_len = min(p.seqused_k[seq], p.max_kv);
  else { k0 = p.cu_k[seq]; kv_len = p.cu_k[seq + 1] - k0; }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  int head_of[QT], i0_of[QT];
  bool any = false;
#pragma unroll
  for (int t = 0; t < QT; t++) {
    const int s = wave * QT + t;
    head_of[t] = hg * hpw + s % hpw;
    i0_of[t] = bx * rows_per_block + 16 * (s / hpw);
    any = any || i0_of[t] < qlen;
  }
  if (qlen <= 0 || kv_len <= 0 || !any) return;
  const int kvh = head_of[0] / (p.Hq / p.Hkv);  // all heads of a block share the kv head
  const int shift = kv_len - qlen;  // absolute position of local row 0

  using Wave = AttnWave<ET, DK, DV, QT, PAD>;
  Wave w;
  w.init_sizes(p);
  int maxpos = -1;
#pragma unroll
  for (int t = 0; t < QT; t++) {
    const int i = i0_of[t] + r16;
    const bool ok = i < qlen;
    const int pos = p.causal ? shift + i : kv_len - 1;
    w.qpos[t] = (ok && pos >= 0) ? pos : -1;
    w.load_q(t, p.q + (int64_t)(q0 + (ok ? i : 0)) * p.sqt + (int64_t)head_of[t] * p.sqh, ok);
    maxpos = max(maxpos, w.qpos[t]);
  }
  // wave-uniform last visible key
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) maxpos = max(maxpos, __shfl_xor(maxpos, o, 64));

  float M[QT], L[QT];
  f32x4 ACC[QT][Wave::NACC];
#pragma unroll
  for (int t = 0; t < QT; t++) {
    M[t] = -INFINITY; L[t] = 0.f;
#pragma unroll
    for (int i = 0; i < Wave::NACC; i++) ACC[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const KVSource<KIND> src = make_source<KIND>(p, seq, kvh, k0, kv_len);
  for (int cs = 0; cs <= maxpos; cs += ATT_CHUNK) {
    w.run_chunk(src, cs, min(cs + ATT_CHUNK, maxpos + 1), kv_len, p.qk_scale);
#pragma unroll
    for (int t = 0; t < QT; t++) {
      float Mn, A, B;
      fold_scales(M[t], w.m[t], Mn, A, B);
      L[t] = fold_add(L[t], A, w.l[t], B);
#pragma unroll
      for (int i = 0; i < Wave::NACC; i++)
#pragma unroll
        for (int r = 0; r < 4; r++) ACC[t][i][r] = fold_add(ACC[t][i][r], A, w.acc[t][i][r], B);
      M[t] = Mn;
    }
  }

#pragma unroll
  for (int t = 0; t < QT; t++) {
    const int i = i0_of[t] + r16;
    if (i >= qlen) continue;
    bf16_t* op = p.o + (int64_t)(q0 + i) * p.sot + (int64_t)head_of[t] * p.soh;
    const bool dead = w.qpos[t] < 0;  // no visible key: define the output as 0
    // (m + log2 l) ln 2, the form the reference saves for its backward (:187-191); +inf for a dead row
    // makes every recomputed probability of that row 0
    if (p.lse && g == 0)
      p.lse[(int64_t)(q0 + i) * p.Hq + head_of[t]] = dead ? INFINITY : (M[t] + __builtin_amdgcn_logf(L[t])) * 0.6931471824645996f;
#pragma unroll
    for (int ds = 0; ds < (DV + 127) / 128; ds++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int d0 = 128 * ds + 32 * g + 8 * r;
        if (d0 < w.dv) {
          uint32_t pk[4];
#pragma unroll
          for (int h = 0; h < 4; h++) {
            const float a = dead ? 0.f : ACC[t][ds * 8 + 2 * h][r] / L[t];
            const float b = dead ? 0.f : ACC[t][ds * 8 + 2 * h + 1][r] / L[t];
            pk[h] = ET::pack2(a, b);
          }
          attn_st8<PAD>(op, d0, make_uint4(pk[0], pk[1], pk[2], pk[3]), w.dv, w.elem);
        }
      }
  }
}

// ---------------------------------------------------------------------------------------
// General kernel for head size 128, K and V through LDS. Same tile slots as attn_prefill_kernel
// (4 wavefronts x 2 query tiles spread over hpw heads of one kv head), but every 64-key block is
// brought in once per workgroup by direct-to-LDS loads (no staging registers) into one of two
// 32 KB stages, and all wavefronts take their operands from there:
//   * rows are 256 bytes; 16-byte piece c of key row r is stored at piece c ^ (r & 15), which makes
//     both kinds of read below conflict free;
//   * S: the A operand (16 keys x 32 dims) is a 16-byte read per lane, as from global memory before;
//   * P V: the A operand (16 dims x 32 keys) comes from two transposing reads (ds_read_b64_tr_b16):
//     the 16 lanes of a group address 4 keys x 16 dims in 8-byte pieces and each lane receives one
//     dim of those 4 keys. Lane (r16, g) of fragment f ends up with dim 16 f + r16 for the keys
//     16 (idx / 4) + 4 g + idx % 4 of k-slot idx = the slot order of P in AttnWave::scores, so no
//     register transposes are needed. The accumulator of fragment f holds dims 16 f + 4 g + r.
// Scores, softmax, chunk folding are the code of AttnWave; each output element sees the same operand
// values in the same MFMA k-slots as in the other attention kernels, so the bits are the same.
// ---------------------------------------------------------------------------------------
typedef short v4s_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

constexpr int PFL_WAVES = 8, PFL_QT = 2, PFL_SLOTS = PFL_WAVES * PFL_QT;  // 16 query tiles per block
constexpr int PFL_STAGE = 2 * ATT_BLOCK * 256;                             // K block, then V block
constexpr int PFL_NS = 3;                                                   // K/V stages in flight
constexpr int PFL_LDS = PFL_NS * PFL_STAGE + PFL_SLOTS * 16 * 256;         // stages + the query tiles = 160 KB

template <int KIND>
__global__ __launch_bounds__(64 * PFL_WAVES) void attn_prefill_lds_kernel(AttnParams p, int hpw) {
  constexpr int D = 128, QT = PFL_QT, KS = D / 32;
  constexpr int KPW = ATT_BLOCK / PFL_WAVES;  // keys of a block that one wavefront brings in
  extern __shared__ __attribute__((aligned(1024))) uint8_t pf_lds[];

  const int rows_per_block = 16 * (PFL_SLOTS / hpw);
  int seq, bx, hg;
  if (!locate_row_block(p, rows_per_block, seq, bx, hg)) return;
  const int q0 = p.cu_q[seq];
  const int qlen = p.cu_q[seq + 1] - q0;
  if (p.single_mode == 2 && qlen == 1) return;  // a decode kernel of the same launch takes these
  int kv_len, k0 = 0;
  if constexpr (KIND != SRC_PACKED) kv_len = min(p.seqused_k[seq], p.max_kv);
  else { k0 = p.cu_k[seq]; kv_len = p.cu_k[seq + 1] - k0; }
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i_base = bx * rows_per_block;
  if (qlen <= 0 || kv_len <= 0 || i_base >= qlen) return;  // uniform over the block
  const int shift = kv_len - qlen;  // absolute position of local row 0
  // last key any row of the block may see (uniform): every wavefront walks the blocks up to it
  const int blk_maxpos = p.causal ? shift + min(i_base + rows_per_block, qlen) - 1 : kv_len - 1;
  if (blk_maxpos < 0) {  // no visible key for any row: outputs are defined as 0
    for (int e = threadIdx.x; e < rows_per_block * hpw * (D / 8); e += 64 * PFL_WAVES) {
      const int row = i_base + e / (hpw * (D / 8)), rem = e % (hpw * (D / 8));
      if (row < qlen)
        *(uint4*)(p.o + (int64_t)(q0 + row) * p.sot + (int64_t)(hg * hpw + rem / (D / 8)) * p.soh +
                  8 * (rem % (D / 8))) = make_uint4(0, 0, 0, 0);
    }
    return;
  }

  int head_of[QT], i0_of[QT];
#pragma unroll
  for (int t = 0; t < QT; t++) {
    const int s = wave * QT + t;
    head_of[t] = hg * hpw + s % hpw;
    i0_of[t] = i_base + 16 * (s / hpw);
  }
  const int kvh = (hg * hpw) / (p.Hq / p.Hkv);

  // ---- this wavefront's query tiles go to its own LDS region (read back every block, which frees
  // 32 registers); piece c of row r at piece c ^ r, like the key rows
  uint8_t* qs = pf_lds + PFL_NS * PFL_STAGE + wave * (QT * 16 * 256);
  int qpos[QT];
#pragma unroll
  for (int t = 0; t < QT; t++) {
    const int i = i0_of[t] + r16;
    const bool ok = i < qlen;
    const int pos = p.causal ? shift + i : kv_len - 1;
    qpos[t] = (ok && pos >= 0) ? pos : -1;
    const bf16_t* qp = p.q + (int64_t)(q0 + (ok ? i : 0)) * p.sqt + (int64_t)head_of[t] * p.sqh + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; s++)
      *(uint4*)(qs + (16 * t + r16) * 256 + (((4 * s + g) ^ r16) * 16)) = ldg16(qp + 32 * s, ok);
  }
  // smallest last-visible key over the rows of each tile (wave-uniform; -1 if a row is not valid):
  // blocks that end at or before it need no masking
  int qpos_min[QT];
#pragma unroll
  for (int t = 0; t < QT; t++) {
    int v = qpos[t];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
    qpos_min[t] = __builtin_amdgcn_readfirstlane(v);  // a scalar register
  }

  float m[QT], l[QT], M[QT], L[QT];
  f32x4 acc[QT][8], ACC[QT][8];
#pragma unroll
  for (int t = 0; t < QT; t++) {
    M[t] = -INFINITY; L[t] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) ACC[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const KVSource<KIND> src = make_source<KIND>(p, seq, kvh, k0, kv_len);
  // ---- loads: wavefront v brings in keys [8 v, 8 v + 8) of a block, K and V, 4 keys (1 KB) per
  // instruction; lane l writes slot l % 16 of its key row and therefore fetches logical piece
  // (l % 16) ^ (row & 15) of K. A transposing read of V touches two adjacent pieces in each of its rows, so
  // there the pair index must differ between the rows read together: V uses (l % 16) ^ 2 (row & 7).
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr_t)pf_lds;
  // The 8 keys a wavefront brings in lie in one 16-key tile (tile wave / 2). For the paged-by-tile and the
  // packed sources the address is therefore a wave-uniform base (scalar registers) plus a small per-lane byte
  // offset, which keeps 64-bit per-lane address arithmetic out of the loop.
  static_assert(KPW == 8, "a wavefront's keys must stay inside one 16-key tile");
  const int ld_tt = wave >> 1;
  int pg_cache = 0, pg_base = -64;  // SRC_FAST: page ids of this wavefront's tile for blocks [pg_base, pg_base + 64), one per lane
  // Per-lane parts of a load's byte offset inside the wavefront's 16-key tile that do not change from block to block:
  // the key's row in the tile and the swizzled 16-byte slot. Per block only the clamp of the row to the sequence's
  // last key and one 32-bit multiply-add per load remain.
  int row_in[KPW / 4];
  uint32_t kslot[KPW / 4], vslot[KPW / 4];
  if constexpr (KIND != SRC_GENERIC) {
#pragma unroll
    for (int j = 0; j < KPW / 4; j++) {
      const int row = KPW * wave + 4 * j + (lane >> 4);
      row_in[j] = row & 15;
      kslot[j] = 16u * (uint32_t)((lane & 15) ^ (row & 15));
      vslot[j] = 16u * (uint32_t)((lane & 15) ^ ((row & 7) << 1));
    }
  }
  auto issue_block = [&](int kb, int stage) {
    const uint32_t dst0 = lds0 + stage * PFL_STAGE + KPW * wave * 256;
    if constexpr (KIND == SRC_GENERIC) {
      const typename KVSource<KIND>::Tiles tl = src.tiles(kb);
#pragma unroll
      for (int j = 0; j < KPW / 4; j++) {
        const int row = KPW * wave + 4 * j + (lane >> 4);  // key row inside the block
        const bool ok = kb + row < kv_len;
        const bf16_t* kp = src.krow(tl, kb, ld_tt, ok ? (row & 15) : 0) + 8 * ((lane & 15) ^ (row & 15));
        const bf16_t* vp = src.vrow(tl, kb, ld_tt, ok ? (row & 15) : 0) + 8 * ((lane & 15) ^ ((row & 7) << 1));
        lds_load16_v(dst0 + 4 * j * 256, kp);
        lds_load16_v(dst0 + 4 * j * 256 + ATT_BLOCK * 256, vp);
      }
    } else {
      // first key of the wavefront's tile, clamped like every key address: a tile that starts past the end
      // is read from the sequence's key 0 (never used), keys past the end inside a tile re-read the last key
      const int tile_key = kb + 16 * ld_tt;
      int key0;
      const bf16_t *kt, *vt;
      if constexpr (KIND == SRC_FAST) {
        key0 = tile_key <= src.last ? tile_key : 0;
        // Page id of the wavefront's tile without a memory round trip per block: lane L keeps the id for block
        // pg_base + L (one vector load per 64 blocks), and the block's id is read from its lane. Fetched per block
        // it cost every wavefront an L2 latency between the barrier and its loads and MFMAs.
        const int b = kb / ATT_BLOCK;
        if (b - pg_base >= 64) {  // wave-uniform
          pg_base = b;
          const int tk = (b + lane) * ATT_BLOCK + 16 * ld_tt;
          pg_cache = src.bt[(tk <= src.last ? tk : 0) >> src.shift];
        }
        const int pg = __builtin_amdgcn_readlane(pg_cache, b - pg_base);
        const int off = key0 & (src.ps - 1);
        kt = src.kbase + (int64_t)pg * src.skb + (int64_t)off * src.skp;
        vt = src.vbase + (int64_t)pg * src.svb + (int64_t)off * src.svp;
      } else {
        key0 = min(tile_key, src.last);
        kt = src.kbase + (int64_t)key0 * src.skp;
        vt = src.vbase + (int64_t)key0 * src.svp;
      }
      const uint64_t kb64 = (uint64_t)kt, vb64 = (uint64_t)vt;
      const uint64_t ksb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(kb64 >> 32)) << 32) |
                           (uint32_t)__builtin_amdgcn_readfirstlane((int)kb64);
      const uint64_t vsb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(vb64 >> 32)) << 32) |
                           (uint32_t)__builtin_amdgcn_readfirstlane((int)vb64);
      // rows past the sequence's last key repeat it (finite data under zero weights); a tile wholly past it reads key 0
      const int last_in = tile_key <= src.last ? src.last - tile_key : 0;  // wave-uniform
#pragma unroll
      for (int j = 0; j < KPW / 4; j++) {
        const uint32_t dk = (uint32_t)min(row_in[j], last_in);  // 0 .. 15
        const uint32_t koff = dk * (uint32_t)(src.skp * 2) + kslot[j];
        const uint32_t voff = dk * (uint32_t)(src.svp * 2) + vslot[j];
        lds_load16_sv(dst0 + 4 * j * 256, koff, (const void*)ksb);
        lds_load16_sv(dst0 + 4 * j * 256 + ATT_BLOCK * 256, voff, (const void*)vsb);
      }
    }
  };

  auto block_compute = [&](int kb, int stage) {
    __builtin_amdgcn_iglp_opt(1);  // scheduling hint: interleave the LDS fragment reads with the MFMAs (measured 3-4 %)
    const uint8_t* ks = pf_lds + stage * PFL_STAGE;
    const uint8_t* vs = ks + ATT_BLOCK * 256;
    // ---- S^T = K Q^T: the key fragments are shared by both query tiles; per accumulator the k-steps
    // run in ascending order as everywhere else
    f32x4 st[QT][4];
#pragma unroll
    for (int t = 0; t < QT; t++)
#pragma unroll
      for (int tt = 0; tt < 4; tt++) st[t][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; s++) {
      uint4 qfr[QT];
#pragma unroll
      for (int t = 0; t < QT; t++) qfr[t] = *(const uint4*)(qs + (16 * t + r16) * 256 + (((4 * s + g) ^ r16) * 16));
#pragma unroll
      for (int tt = 0; tt < 4; tt++) {
        const int row = 16 * tt + r16;
        const uint4 kfr = *(const uint4*)(ks + row * 256 + (((4 * s + g) ^ (row & 15)) * 16));
#pragma unroll
        for (int t = 0; t < QT; t++) st[t][tt] = mfma16(kfr, qfr[t], st[t][tt]);
      }
    }
    uint4 pf[QT][2];
#pragma unroll
    for (int t = 0; t < QT; t++)
      attn_softmax_tile<ElemBF16>(st[t], kb, p.qk_scale, qpos[t], m[t], l[t], acc[t], pf[t], kb + ATT_BLOCK - 1 <= qpos_min[t]);
    // ---- P V. For k-slots idx = 0..3 (first read) and 4..7 (second) of 32-key chunk ch, addressing
    // lane i = r16 of group g points at key 32 ch + 16 (idx / 4) + 4 g + i / 4, dims 16 f + 4 (i % 4) .. +3
#pragma unroll
    for (int ch = 0; ch < 2; ch++) {
#pragma unroll
      for (int f = 0; f < 8; f++) {
        const int byte = 32 * f + 8 * (r16 & 3);
        const int row_lo = 32 * ch + 4 * g + (r16 >> 2), row_hi = row_lo + 16;
        const v4s_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) v4s_t*)(vs + row_lo * 256 + (((byte >> 4) ^ ((row_lo & 7) << 1)) * 16) + (byte & 15)));
        const v4s_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) v4s_t*)(vs + row_hi * 256 + (((byte >> 4) ^ ((row_hi & 7) << 1)) * 16) + (byte & 15)));
        const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
        const uint4 vf = make_uint4(lo2.x, lo2.y, hi2.x, hi2.y);
#pragma unroll
        for (int t = 0; t < QT; t++) acc[t][f] = mfma16(vf, pf[t][ch], acc[t][f]);
      }
    }
  };

  const int nblk = blk_maxpos / ATT_BLOCK + 1;
  auto chunk_reset = [&](int kb) {
    if ((kb & (ATT_CHUNK - 1)) == 0) {
#pragma unroll
      for (int t = 0; t < QT; t++) {
        m[t] = -INFINITY; l[t] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) acc[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
    }
  };
  auto chunk_fold = [&](int kb, int b) {
    if (((kb + ATT_BLOCK) & (ATT_CHUNK - 1)) == 0 || b + 1 == nblk) {
#pragma unroll
      for (int t = 0; t < QT; t++) {
        float Mn, A, B;
        fold_scales(M[t], m[t], Mn, A, B);
        L[t] = fold_add(L[t], A, l[t], B);
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
          for (int r = 0; r < 4; r++) ACC[t][i][r] = fold_add(ACC[t][i][r], A, acc[t][i][r], B);
        M[t] = Mn;
      }
    }
  };
  // one barrier per block: passing it says that block b has landed for everyone and that everyone
  // is done with block b - 1, whose stage then takes block b + PFL_NS - 1
#pragma unroll
  for (int i = 0; i < PFL_NS - 1; i++)
    if (i < nblk) issue_block(i * ATT_BLOCK, i);
  int stage = 0;
  for (int b0 = 0; b0 < nblk; b0 += ATT_CHUNK / ATT_BLOCK) {  // one chunk of keys: per-chunk state, then the fold
    chunk_reset(b0 * ATT_BLOCK);
    const int b1 = min(nblk, b0 + ATT_CHUNK / ATT_BLOCK);
    for (int b = b0; b < b1; b++) {
      const int kb = b * ATT_BLOCK;
      // KPW / 2 loads per block and wavefront; the next block's may still be in flight
      if (b + 1 < nblk) {
        static_assert(KPW == 8, "the wait below counts 4 loads per block and wavefront");
        asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      __syncthreads();
      if (b + PFL_NS - 1 < nblk) issue_block(kb + (PFL_NS - 1) * ATT_BLOCK, stage == 0 ? PFL_NS - 1 : stage - 1);
      block_compute(kb, stage);
      stage = stage + 1 == PFL_NS ? 0 : stage + 1;
    }
    chunk_fold((b1 - 1) * ATT_BLOCK, b1 - 1);
  }

  // lane (r16 = query row, g) holds dims 16 f + 4 g + r of fragment f
#pragma unroll
  for (int t = 0; t < QT; t++) {
    const int i = i0_of[t] + r16;
    if (i >= qlen) continue;
    bf16_t* op = p.o + (int64_t)(q0 + i) * p.sot + (int64_t)head_of[t] * p.soh;
    const bool dead = qpos[t] < 0;
    if (p.lse && g == 0)
      p.lse[(int64_t)(q0 + i) * p.Hq + head_of[t]] = dead ? INFINITY : (M[t] + __builtin_amdgcn_logf(L[t])) * 0.6931471824645996f;
#pragma unroll
    for (int f = 0; f < 8; f++) {
      uint2 pk;
      pk.x = pack_bf16x2(dead ? 0.f : ACC[t][f][0] / L[t], dead ? 0.f : ACC[t][f][1] / L[t]);
      pk.y = pack_bf16x2(dead ? 0.f : ACC[t][f][2] / L[t], dead ? 0.f : ACC[t][f][3] / L[t]);
      *(uint2*)(op + 16 * f + 4 * g) = pk;
    }
  }
}

// Which decode form a launch takes: chunks folded inside one workgroup per (sequence, kv head) when that
// fills the machine (or mode 4), else one wavefront per chunk plus a combine launch (or mode 3); only the
// latter uses the workspace. A function of the shapes alone. Returns 1 = fused, 0 = split, < 0 = error.
static inline int decode_form(int mode, int64_t num_seqs, int Hq, int Hkv, int Dv_caller) {
  // the value head size the kernels are built for: every caller of this function (workspace queries with the
  // caller's size, launches with the built-for size) must reach the same answer
  const int Dv = Dv_caller <= 32 ? 32 : Dv_caller <= 64 ? 64 : Dv_caller <= 128 ? 128 : 256;
  const int G = Hq / Hkv;
  if (G > 32) return VX_ERR_UNSUPPORTED;
  const int QT = G <= 16 ? 1 : 2, NW = G <= 16 ? 8 : 4;
  const int64_t lds = ((int64_t)NW * (QT * ((Dv + 127) / 128) * 8 + QT) * 64 + 16 * QT * (Dv / 4)) * 16 + 16 * QT * (Dv / 4) * 8;
  const bool fits = lds <= 160 * 1024;
  if (mode == 4 && !fits) return VX_ERR_UNSUPPORTED;
  // One workgroup per CU is enough for the fused form (measured at 256 workgroups, 64 sequences x 4 kv heads and
  // 32 x 8: 13-19 % ahead of the split form on contexts of 256..2048 and 1000..8192 tokens; at 128 workgroups level on
  // short contexts and 25 % behind on long ones).
  return (mode == 4 || (mode == 0 && fits && num_seqs * Hkv >= 256)) ? 1 : 0;
}

template <class ET, int DK, int DV, bool PAD>
static int launch_attn(const AttnParams& p_in, int mode, int max_q, int total_q, hipStream_t stream) {
  AttnParams p = p_in;
  const bool fast = p.page_shift >= 4;  // page size a power of two >= 16
  // A general paged launch hands its sequences of one query row (decode tokens that share the batch with prefill
  // chunks, or a whole decode batch that a caller launches with the bucket's token count as max_seqlen_q) to the
  // fused decode kernel and gives the general kernel the rest: the same bits (a prefill row equals the decode step
  // of that token), a fraction of the work. Needs the fused form (chunk states in LDS, no workspace) and no lse.
  const bool hybrid = mode == 1 && !p.lse && max_q != 1 && decode_form(4, p.num_seqs, p.Hq, p.Hkv, DV) == 1;
  if (hybrid) {
    AttnParams d = p;
    d.single_mode = 1;  // seq_order, if given, orders these decode workgroups
    const int64_t max_kv = p.max_kv;
    d.max_chunks = (int)((max_kv + ATT_CHUNK - 1) / ATT_CHUNK);
    const int rc = launch_attn<ET, DK, DV, PAD>(d, 4, 1, total_q, stream);
    if (rc != VX_OK) return rc;
    p.single_mode = 2;
  }
  if (mode == 0 || mode == 3 || mode == 4) {
    const int G = p.Hq / p.Hkv;
    constexpr int NW1 = 8, NW1S = 4, NW2 = 4;  // wavefronts per block for one (many / very many workgroups) / two q-tiles
    static_assert(fused_lds_bytes<DV, 1, NW1>() == ((int64_t)NW1 * (((DV + 127) / 128) * 8 + 1) * 64 + 16 * (DV / 4)) * 16 + 16 * (DV / 4) * 8,
                  "decode_form() restates fused_lds_bytes");
    const int form = decode_form(mode, p.num_seqs, p.Hq, p.Hkv, DV);
    if (form < 0) return form;
    const bool fused = form == 1;
    if (fused) {
      const dim3 grid(p.Hkv, p.num_seqs);
#define VX_FUSED(KERNEL, QTV, KINDV, NW)                                                             \
  do {                                                                                             \
    constexpr int LDSB = fused_lds_bytes<DV, QTV, NW>();                                           \
    static DeviceOnce once;                                                                        \
    const int dev = once.slot();                                                                   \
    if (once.need(dev)) {                                                                          \
      if (hipFuncSetAttribute((const void*)KERNEL<ET, DK, DV, QTV, KINDV, NW, PAD>,                \
                              hipFuncAttributeMaxDynamicSharedMemorySize, LDSB) != hipSuccess) {   \
        (void)hipGetLastError();                                                                   \
        return VX_ERR_LAUNCH;                                                                      \
      }                                                                                            \
      once.mark(dev);                                                                              \
    }                                                                                              \
    KERNEL<ET, DK, DV, QTV, KINDV, NW, PAD><<<grid, 64 * NW, LDSB, stream>>>(p);                   \
  } while (0)
      if (G <= 16) {
        if constexpr (DK <= 128 && DV <= 128) {
          // With >= 1024 workgroups, 4 wavefronts each: two workgroups then share a CU and one's set-up
          // and fold overlap the other's streaming (measured 121.5 vs 124.8 us at 256 sequences x 4 kv
          // heads; with 512 workgroups of long sequences 8 wavefronts are faster, 115 vs 125 us).
          if ((int64_t)p.num_seqs * p.Hkv >= 1024) {
            if (fast) VX_FUSED(attn_decode_fused_kernel_occ2, 1, SRC_FAST, NW1S);
            else VX_FUSED(attn_decode_fused_kernel_occ2, 1, SRC_GENERIC, NW1S);
          } else if (fast) VX_FUSED(attn_decode_fused_kernel_occ2, 1, SRC_FAST, NW1);
          else VX_FUSED(attn_decode_fused_kernel_occ2, 1, SRC_GENERIC, NW1);
        } else {
          if (fast) VX_FUSED(attn_decode_fused_kernel, 1, SRC_FAST, NW1);
          else VX_FUSED(attn_decode_fused_kernel, 1, SRC_GENERIC, NW1);
        }
      } else {
        if (fast) VX_FUSED(attn_decode_fused_kernel, 2, SRC_FAST, NW2);
        else VX_FUSED(attn_decode_fused_kernel, 2, SRC_GENERIC, NW2);
      }
#undef VX_FUSED
      return launch_status();
    }
    dim3 grid(p.Hkv, p.num_seqs, p.max_chunks);
    if (G <= 16) {
      if constexpr (DK <= 128 && DV <= 128) {
        if (fast) attn_decode_split_kernel_occ2<ET, DK, DV, 1, SRC_FAST, PAD><<<grid, 64, 0, stream>>>(p);
        else attn_decode_split_kernel_occ2<ET, DK, DV, 1, SRC_GENERIC, PAD><<<grid, 64, 0, stream>>>(p);
      } else {
        if (fast) attn_decode_split_kernel<ET, DK, DV, 1, SRC_FAST, PAD><<<grid, 64, 0, stream>>>(p);
        else attn_decode_split_kernel<ET, DK, DV, 1, SRC_GENERIC, PAD><<<grid, 64, 0, stream>>>(p);
      }
    } else {
      if (fast) attn_decode_split_kernel<ET, DK, DV, 2, SRC_FAST, PAD><<<grid, 64, 0, stream>>>(p);
      else attn_decode_split_kernel<ET, DK, DV, 2, SRC_GENERIC, PAD><<<grid, 64, 0, stream>>>(p);
    }
    if (G <= 16) attn_decode_combine_kernel<ET, DV, 1, PAD><<<dim3(p.Hkv, p.num_seqs), 64, 0, stream>>>(p);
    else attn_decode_combine_kernel<ET, DV, 2, PAD><<<dim3(p.Hkv, p.num_seqs), 64, 0, stream>>>(p);
  } else {
    constexpr int QT = (DK > 128) ? 1 : 2;
    const int rows = max_q > 0 ? max_q : total_q;
    // query heads of one kv head that share a block (a divisor of the group size and of the 4 * QT
    // tile slots)
    const int G = p.Hq / p.Hkv;
    int hpw = 1;
    while (hpw * 2 <= 4 * QT && G % (hpw * 2) == 0) hpw *= 2;
    const int rpb = 16 * (4 * QT / hpw);
    // (sequence, row block) pairs: the plain grid of ceil(rows / rpb) x num_seqs, or the compact numbering when
    // that is smaller (sequences with very different numbers of query rows)
    auto row_grid = [&](int rb, unsigned heads) {
      const int64_t blocks = (rows + rb - 1) / rb;
      const int64_t plain = blocks * p.num_seqs;
      const int64_t comp = (int64_t)total_q / rb + p.num_seqs;
      p.compact = (comp < plain || blocks > 65535 || p.num_seqs > 65535) ? 1 : 0;  // grid.y and grid.z end at 65535
      if (p.compact && comp <= 65535) return dim3(heads, (unsigned)comp, 1);
      if (p.compact) {
        p.compact = 2;
        return dim3((unsigned)comp, heads, 1);
      }
      // eight consecutive workgroup ids = the head groups of 8 / heads sequences at one row block (measured on 4 head
      // groups: 1 / 2 / 4 / 8 sequences give 135 / 115 / 111 / 111 us on 8 x 1024-token prompts and 555 / 554 / 622 /
      // 868 us on 512-token chunks behind prefixes up to 8192, where more sequences in flight share less of the L2)
      p.grid_heads = (int)heads;
      p.grid_sg = std::max(1, std::min(p.num_seqs, (int)(8u / std::max(1u, heads))));
      return dim3(heads * (unsigned)p.grid_sg, (unsigned)blocks, (unsigned)((p.num_seqs + p.grid_sg - 1) / p.grid_sg));
    };
    dim3 grid = row_grid(rpb, (unsigned)(p.Hq / hpw));
    if constexpr (DK == 128 && DV == 128 && !PAD && ET::kDtype == 0) {
      // K and V through LDS, shared by the 16 query tiles of a block
      int hp = 1;
      while (hp * 2 <= 8 && G % (hp * 2) == 0) hp *= 2;
      const int rb = 16 * (PFL_SLOTS / hp);
      const dim3 lgrid = row_grid(rb, (unsigned)(p.Hq / hp));
      static DeviceOnce once;
      const int dev = once.slot();
      if (once.need(dev)) {
        if (hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<SRC_PACKED>, hipFuncAttributeMaxDynamicSharedMemorySize, PFL_LDS) != hipSuccess ||
            hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<SRC_FAST>, hipFuncAttributeMaxDynamicSharedMemorySize, PFL_LDS) != hipSuccess ||
            hipFuncSetAttribute((const void*)attn_prefill_lds_kernel<SRC_GENERIC>, hipFuncAttributeMaxDynamicSharedMemorySize, PFL_LDS) != hipSuccess) {
          (void)hipGetLastError();
          return VX_ERR_LAUNCH;
        }
        once.mark(dev);
      }
      if (mode == 2) attn_prefill_lds_kernel<SRC_PACKED><<<lgrid, 64 * PFL_WAVES, PFL_LDS, stream>>>(p, hp);
      else if (fast) attn_prefill_lds_kernel<SRC_FAST><<<lgrid, 64 * PFL_WAVES, PFL_LDS, stream>>>(p, hp);
      else attn_prefill_lds_kernel<SRC_GENERIC><<<lgrid, 64 * PFL_WAVES, PFL_LDS, stream>>>(p, hp);
      return launch_status();
    }
    if (mode == 2) attn_prefill_kernel<ET, DK, DV, QT, SRC_PACKED, PAD><<<grid, 256, 0, stream>>>(p, hpw);
    else if (fast) attn_prefill_kernel<ET, DK, DV, QT, SRC_FAST, PAD><<<grid, 256, 0, stream>>>(p, hpw);
    else attn_prefill_kernel<ET, DK, DV, QT, SRC_GENERIC, PAD><<<grid, 256, 0, stream>>>(p, hpw);
  }
  return launch_status();
}

// Launchers that live in translation units of their own (compile time): bf16 on padded head sizes and fp16 (always
// through the padded code). DKb / DVb: the built-for sizes, one of (64, 64), (128, 128), (256, 128), (256, 256).
int launch_attn_bf16_padded(const AttnParams& p, int DKb, int DVb, int mode, int max_q, int total_q, hipStream_t stream);
int launch_attn_f16(const AttnParams& p, int DKb, int DVb, int mode, int max_q, int total_q, hipStream_t stream);

}  // namespace vx
