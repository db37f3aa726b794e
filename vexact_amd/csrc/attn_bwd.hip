// Backward of causal varlen attention on packed q / k / v (the training-side twin of the rollout
// attention): dQ, dK, dV from dO and the forward's log-sum-exp. Replaces _varlen_attn_bwd_dq_kernel
// and _varlen_attn_bwd_dkv_kernel (vexact/batch_invariant_ops/triton_invariant_attention.py:193-430),
// same formulas and the same bf16 roundings of P and dS before they enter a matrix product:
//   P_ij  = exp(scale * q_i.k_j - lse_i) for visible keys, else 0
//   dP_ij = dO_i . v_j ;  delta_i = O_i . dO_i ;  dS_ij = P_ij (dP_ij - delta_i) scale
//   dQ_i = sum_j r16(dS_ij) k_j ;  dK_j = sum_i r16(dS_ij) q_i ;  dV_j = sum_i r16(P_ij) dO_i
//
// Both kernels are one routine seen from two sides. A wavefront keeps a 16-row "stationary" tile
// (queries for dQ, keys for dK / dV) as MFMA B operands and walks the other side in 64-row blocks:
//   scores  D[moving row][stationary col] = A(moving rows, 16 x 32 dims) x B(stationary, 32 dims x 16)
// so a lane ends up with four consecutive moving rows of one stationary column: exactly the k-slot
// order an MFMA B operand wants once two 16-row tiles are paired. The products that contract over
// the moving rows (dQ += K^T dS^T, dK += Q^T dS, dV += dO^T P) therefore take P / dS straight from
// the accumulator registers, and their A operands (the moving rows transposed) come from 16-byte
// row loads and an 8 x 8 bf16 transpose in registers. Every sum runs in a fixed order that depends
// only on the sequence's own lengths, so a sequence's gradients do not depend on the batch.
#include "attn_bwd_core.h"
#include "attn_f32_launch.h"

namespace vx {

// ---------------------------------------------------------------------------------------
// Head size 128: the moving side goes through LDS once per workgroup. 8 wavefronts hold 8 stationary
// tiles (128 queries of one head for dQ); every 64-row block of the two moving arrays (K and V) is
// brought in by direct-to-LDS loads into one of two 32 KB stages while the previous block is being
// used. Rows are 256 bytes with 16-byte piece c of row r stored at piece c ^ bwl_swz(r): the 16-byte
// fragment reads (A operands of the score products) and the transposing 8-byte reads
// (ds_read_b64_tr_b16, A operands of the products that contract over the moving rows) are both
// free of bank conflicts, and the transposing reads deliver the rows in the k-slot order in which
// P / dS sit in the accumulator registers, so there are no register transposes.
// The accumulator of fragment f holds dims 16 f + 4 g + r of the lane's stationary row.
// ---------------------------------------------------------------------------------------
constexpr int BWL_WAVES = 8;
constexpr int BWL_ARR = 64 * 256;          // one 64-row array
constexpr int BWL_STAGE = 2 * BWL_ARR;     // two arrays per stage
constexpr int BWL_LDS = 2 * BWL_STAGE;     // two stages
typedef short bw_v4s_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* bw_lds_ptr_t;
// A 16-byte fragment read takes one piece from each of 16 consecutive rows: the swizzle term must differ over
// them. A transposing read takes two adjacent pieces from each of 8 consecutive rows at a time: the term
// without its lowest bit must differ over those.
__device__ __forceinline__ int bwl_swz(int row) { return ((row & 7) << 1) | ((row >> 3) & 1); }

// wavefront `wave` of NW brings rows [64 / NW * wave, +64 / NW) of a 64-row array into LDS: 4 rows per instruction
template <int NW = BWL_WAVES>
__device__ __forceinline__ void bwl_issue_rows(const bf16_t* base, int64_t row_stride, int first_row, int last_row,
                                               uint32_t lds_arr, int wave) {
  const int lane = threadIdx.x & 63;
  constexpr int RPW = 64 / NW;
  // wave-uniform base (scalar registers) + 32-bit lane offset: rows past the end re-read the last row
  const int r0 = min(first_row, last_row);
  const uint64_t b64 = (uint64_t)(base + (int64_t)r0 * row_stride);
  const uint64_t sb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(b64 >> 32)) << 32) |
                      (uint32_t)__builtin_amdgcn_readfirstlane((int)b64);
#pragma unroll
  for (int j = 0; j < RPW / 4; j++) {
    const int row = RPW * wave + 4 * j + (lane >> 4);
    const int piece = (lane & 15) ^ bwl_swz(row);
    const uint32_t voff = (uint32_t)(min(first_row + row, last_row) - r0) * (uint32_t)(row_stride * 2) + 16u * (uint32_t)piece;
    const uint32_t dst = lds_arr + (RPW * wave + 4 * j) * 256;
    lds_load16_sv(dst, voff, (const void*)sb);
  }
}
// A operand of a score product: row 16 tt + r16 of the array, dims 32 s + 8 g .. +8
__device__ __forceinline__ uint4 bwl_frag(const uint8_t* arr, int tt, int s) {
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int row = 16 * tt + r16;
  return *(const uint4*)(arr + row * 256 + (((4 * s + g) ^ bwl_swz(row)) * 16));
}
// acc[f] (rows = dims 16 f + .., cols = stationary) += (array rows, transposed) x pf
__device__ __forceinline__ void bwl_tr_product(const uint8_t* arr, const uint4 (&pf)[2], f32x4 (&acc)[8]) {
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
#pragma unroll
  for (int ch = 0; ch < 2; ch++) {
#pragma unroll
    for (int f = 0; f < 8; f++) {
      const int byte = 32 * f + 8 * (r16 & 3);
      const int row_lo = 32 * ch + 4 * g + (r16 >> 2), row_hi = row_lo + 16;
      const bw_v4s_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) bw_v4s_t*)(arr + row_lo * 256 + (((byte >> 4) ^ bwl_swz(row_lo)) * 16) + (byte & 15)));
      const bw_v4s_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) bw_v4s_t*)(arr + row_hi * 256 + (((byte >> 4) ^ bwl_swz(row_hi)) * 16) + (byte & 15)));
      const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
      acc[f] = mfma16(make_uint4(lo2.x, lo2.y, hi2.x, hi2.y), pf[ch], acc[f]);
    }
  }
}
// lane (g, c): acc[f][r] = element (dim 16 f + 4 g + r) of stationary row c
__device__ __forceinline__ void bwl_store_tile(const f32x4 (&acc)[8], bf16_t* rowp) {
  const int g = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int f = 0; f < 8; f++) {
    uint2 pk;
    pk.x = pack_bf16x2(acc[f][0], acc[f][1]);
    pk.y = pack_bf16x2(acc[f][2], acc[f][3]);
    *(uint2*)(rowp + 16 * f + 4 * g) = pk;
  }
}

// dQ, head size 128: grid (ceil(max_q / 128), Hq, sequences), 512 threads
__global__ __launch_bounds__(64 * BWL_WAVES) void attn_bwd_dq_lds_kernel(AttnBwdParams p) {
  constexpr int KS = 4;
  extern __shared__ __attribute__((aligned(1024))) uint8_t bw_lds[];
  // grid: heads x query tiles x sequences. Workgroup ids go round the eight XCDs and are dispatched in order, so the
  // fastest index holds what has equal work (the heads) and the tile runs downwards: a sequence's tiles that see the
  // most keys start first, its short ones fill the tail. (Which workgroup computes a tile changes no result.)
  const int seq = blockIdx.z, h = blockIdx.x;
  const int q0 = p.cu_q[seq], qlen = p.cu_q[seq + 1] - q0;
  const int k0 = p.cu_k[seq], kv_len = p.cu_k[seq + 1] - k0;
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i_base = (int)(gridDim.y - 1 - blockIdx.y) * (16 * BWL_WAVES);
  if (i_base >= qlen || kv_len <= 0) return;  // uniform over the block
  const int kvh = h / (p.Hq / p.Hkv);
  const int shift = kv_len - qlen;
  // last key any query of the block sees (uniform): every wavefront walks the blocks up to it
  const int blk_maxpos = min(shift + min(i_base + 16 * BWL_WAVES, qlen) - 1, kv_len - 1);
  const int i = i_base + 16 * wave + r16;       // this lane's query
  const bool qok = i < qlen;
  const int pos = qok ? shift + i : -1;
  const int64_t tq = q0 + (qok ? i : qlen - 1);
  uint4 qf[KS], of[KS];
  {
    const bf16_t* qp = p.q + tq * p.sqt + (int64_t)h * p.sqh + 8 * g;
    const bf16_t* dp = p.d_o + tq * p.sdt + (int64_t)h * p.sdh + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; s++) {
      qf[s] = ldg16_raw(qp + 32 * s);
      of[s] = ldg16_raw(dp + 32 * s);
    }
  }
  const float c2 = p.scale * 1.44269504f;
  const float lse2 = p.lse[tq * p.Hq + h] * 1.44269504f;
  const float delta = p.delta[tq * p.Hq + h];
  int wave_maxpos = pos, wave_minpos = pos;  // last key this wavefront's queries see; first row's limit (-1: a row is missing)
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    wave_maxpos = max(wave_maxpos, __shfl_xor(wave_maxpos, o, 64));
    wave_minpos = min(wave_minpos, __shfl_xor(wave_minpos, o, 64));
  }
  wave_maxpos = __builtin_amdgcn_readfirstlane(wave_maxpos);
  wave_minpos = __builtin_amdgcn_readfirstlane(wave_minpos);
  f32x4 acc[8];
#pragma unroll
  for (int f = 0; f < 8; f++) acc[f] = f32x4{0.f, 0.f, 0.f, 0.f};
  // the registers above must be loaded before the first direct-to-LDS load is counted
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  const bf16_t* kb_ = p.k + (int64_t)k0 * p.skt + (int64_t)kvh * p.skh;
  const bf16_t* vb_ = p.v + (int64_t)k0 * p.svt + (int64_t)kvh * p.svh;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(bw_lds_ptr_t)bw_lds;
  auto issue_block = [&](int kb, int stage) {
    bwl_issue_rows(kb_, p.skt, kb, kv_len - 1, lds0 + stage * BWL_STAGE, wave);
    bwl_issue_rows(vb_, p.svt, kb, kv_len - 1, lds0 + stage * BWL_STAGE + BWL_ARR, wave);
  };
  if (blk_maxpos >= 0) issue_block(0, 0);
  auto one_block = [&](int kb, const int stage) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // block kb is in LDS for everyone; everyone is done with the other stage
    if (kb + 64 <= blk_maxpos) issue_block(kb + 64, stage ^ 1);
    if (kb > wave_maxpos) return;  // nothing visible to this wavefront any more (it keeps loading and syncing)
    const uint8_t* ks = bw_lds + stage * BWL_STAGE;
    const uint8_t* vs = ks + BWL_ARR;
    const bool all_visible = kb + 63 <= wave_minpos;  // uniform: no key of the block is masked for any row
    float ds[4][4];
#pragma unroll
    for (int tt = 0; tt < 4; tt++) {
      f32x4 st = f32x4{0.f, 0.f, 0.f, 0.f}, dp = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; s++) {
        st = mfma16(bwl_frag(ks, tt, s), qf[s], st);
        dp = mfma16(bwl_frag(vs, tt, s), of[s], dp);
      }
      if (all_visible) {
#pragma unroll
        for (int r = 0; r < 4; r++)
          ds[tt][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(st[r], c2, -lse2)) * (dp[r] - delta) * p.scale;
      } else {
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int key = kb + 16 * tt + 4 * g + r;
          const float pr = (key <= pos) ? __builtin_amdgcn_exp2f(__builtin_fmaf(st[r], c2, -lse2)) : 0.f;
          ds[tt][r] = pr * (dp[r] - delta) * p.scale;
        }
      }
    }
    uint4 pf[2];
    bwd_pack<ElemBF16>(ds, pf);
    bwl_tr_product(ks, pf, acc);
  };
  // (unrolling over the two stages would make the LDS offsets immediates but costs 13 registers, which
  // takes the kernel over 128 and halves the wavefronts per SIMD)
  for (int kb = 0, stage = 0; kb <= blk_maxpos; kb += 64, stage ^= 1) one_block(kb, stage);
  if (qok) bwl_store_tile(acc, p.dq + tq * p.sdqt + (int64_t)h * p.sdqh);
}

// dK, dV, head size 128: grid (ceil(max_k / (16 NW)), Hkv, sequences), NW wavefronts. The moving side is
// the queries of the kv head's query heads, one head after the other: Q and dO blocks plus the
// 64 rows' lse and delta per stage.
constexpr int BWK_STAGE = 2 * BWL_ARR + 1024;  // Q, dO, then 64 lse and 64 delta values
constexpr int BWK_LDS = 2 * BWK_STAGE;
constexpr int BWK_WAVES = 8;  // 128 keys per workgroup (64-key workgroups: 519 vs 493 us on 8 x 1024 tokens, 5 % ahead on 32 x 1024 and 16 x 2048, 3 % behind on 4 x 4096)

template <int NW>
__global__ __launch_bounds__(64 * NW) void attn_bwd_dkv_lds_kernel(AttnBwdParams p) {
  constexpr int KS = 4;
  extern __shared__ __attribute__((aligned(1024))) uint8_t bw_lds[];
  // grid: (kv heads x sg sequences) x key tiles x groups of sequences, eight workgroup ids (one per XCD) of equal work
  // in the fastest index; the key tile runs upwards: the tiles that every query sees start first. (With the key tile
  // in blockIdx.x, 8 / 16 / 32 tiles per sequence pinned each tile number to one XCD. Measured against that form, 32 /
  // 4 heads: 8 x 1024 tokens 517 -> 493 us, 32 x 1024 2185 -> 1697, 16 x 2048 3901 -> 2779, 4 x 4096 3728 -> 2245;
  // the tile number merely rotated by head and sequence gives 1608 / 2624 / 3370 on the last three.)
  const int kvh = (int)(blockIdx.x % p.Hkv), seq = (int)(blockIdx.z * (gridDim.x / p.Hkv) + blockIdx.x / p.Hkv);
  if (seq >= p.num_seqs) return;  // uniform over the block
  const int q0 = p.cu_q[seq], qlen = p.cu_q[seq + 1] - q0;
  const int k0 = p.cu_k[seq], kv_len = p.cu_k[seq + 1] - k0;
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j_base = (int)blockIdx.y * (16 * NW);
  if (j_base >= kv_len) return;  // uniform over the block
  const int G = p.Hq / p.Hkv;
  const int shift = kv_len - qlen;
  const int j0 = j_base + 16 * wave;            // first key of this wavefront's tile
  const int j = j0 + r16;                       // this lane's key
  const bool kok = j < kv_len;
  const int64_t tk = k0 + (kok ? j : kv_len - 1);
  uint4 kf[KS], vf[KS];
  {
    const bf16_t* kp = p.k + tk * p.skt + (int64_t)kvh * p.skh + 8 * g;
    const bf16_t* vp = p.v + tk * p.svt + (int64_t)kvh * p.svh + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; s++) {
      kf[s] = ldg16_raw(kp + 32 * s);
      vf[s] = ldg16_raw(vp + 32 * s);
    }
  }
  const float c2 = p.scale * 1.44269504f;
  f32x4 dk[8], dv[8];
#pragma unroll
  for (int f = 0; f < 8; f++) {
    dk[f] = f32x4{0.f, 0.f, 0.f, 0.f};
    dv[f] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // first query that sees the block's first key; the moving blocks start there
  const int ib0 = max(0, j_base - shift);
  const int nblk = qlen > ib0 ? (qlen - ib0 + 63) / 64 : 0;
  const int nsteps = nblk * G;  // query heads one after the other
  const uint32_t lds0 = (uint32_t)(uintptr_t)(bw_lds_ptr_t)bw_lds;
  auto issue_step = [&](int step, int stage) {
    const int h = kvh * G + step / nblk, ib = ib0 + 64 * (step % nblk);
    const uint32_t sb = lds0 + stage * BWK_STAGE;
    bwl_issue_rows<NW>(p.q + (int64_t)q0 * p.sqt + (int64_t)h * p.sqh, p.sqt, ib, qlen - 1, sb, wave);
    bwl_issue_rows<NW>(p.d_o + (int64_t)q0 * p.sdt + (int64_t)h * p.sdh, p.sdt, ib, qlen - 1, sb + BWL_ARR, wave);
    if (wave < 2) {  // 64 lse values (wavefront 0) and 64 delta values (wavefront 1), one dword per lane
      const float* src = (wave == 0 ? p.lse : p.delta) + (int64_t)(q0 + min(ib + lane, qlen - 1)) * p.Hq + h;
      const uint32_t dst = sb + 2 * BWL_ARR + wave * 256;
      lds_load4_v(dst, src);
    }
  };
  if (nsteps > 0) issue_step(0, 0);
  const bool tile_full = j0 + 15 < kv_len;  // uniform: every key of this wavefront's tile exists
  auto one_step = [&](int step, const int stage) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // this step's rows are in LDS for everyone; everyone is done with the other stage
    if (step + 1 < nsteps) issue_step(step + 1, stage ^ 1);
    const int ib = ib0 + 64 * (step % nblk);
    if (ib + 63 + shift < j0) return;  // none of the block's queries sees any key of this wavefront's tile
    const uint8_t* qs = bw_lds + stage * BWK_STAGE;
    const uint8_t* os = qs + BWL_ARR;
    const float* lse_s = (const float*)(os + BWL_ARR);
    const float* del_s = lse_s + 64;
    // uniform: all 64 queries exist and even the first of them sees the tile's last key
    const bool all_visible = tile_full && ib + 63 < qlen && j0 + 15 <= shift + ib;
    float pr[4][4], ds[4][4];
#pragma unroll
    for (int tt = 0; tt < 4; tt++) {
      f32x4 st = f32x4{0.f, 0.f, 0.f, 0.f}, dp = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; s++) {
        st = mfma16(bwl_frag(qs, tt, s), kf[s], st);
        dp = mfma16(bwl_frag(os, tt, s), vf[s], dp);
      }
      const float4 l4 = *(const float4*)(lse_s + 16 * tt + 4 * g);
      const float4 d4 = *(const float4*)(del_s + 16 * tt + 4 * g);
      const float lr[4] = {l4.x, l4.y, l4.z, l4.w}, dr[4] = {d4.x, d4.y, d4.z, d4.w};
      if (all_visible) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(st[r], c2, -(lr[r] * 1.44269504f)));
          pr[tt][r] = e;
          ds[tt][r] = e * (dp[r] - dr[r]) * p.scale;
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int iq = ib + 16 * tt + 4 * g + r;  // this register's query (moving row)
          const bool ok = iq < qlen && kok && j <= shift + iq;
          const float e = ok ? __builtin_amdgcn_exp2f(__builtin_fmaf(st[r], c2, -(lr[r] * 1.44269504f))) : 0.f;
          pr[tt][r] = e;
          ds[tt][r] = e * (dp[r] - dr[r]) * p.scale;
        }
      }
    }
    uint4 pfp[2], pfs[2];
    bwd_pack<ElemBF16>(pr, pfp);
    bwd_pack<ElemBF16>(ds, pfs);
    bwl_tr_product(os, pfp, dv);
    bwl_tr_product(qs, pfs, dk);
  };
  for (int step = 0; step < nsteps; step += 2) {
    one_step(step, 0);
    if (step + 1 < nsteps) one_step(step + 1, 1);
  }
  if (kok) {
    bwl_store_tile(dk, p.dk + tk * p.sdkt + (int64_t)kvh * p.sdkh);
    bwl_store_tile(dv, p.dv + tk * p.sdvt + (int64_t)kvh * p.sdvh);
  }
}

// bf16, head size 128 exactly: the LDS kernels
static int launch_attn_bwd_lds128(const AttnBwdParams& p, int64_t total_q, int num_seqs, int max_q, int max_k, hipStream_t stream) {
  attn_bwd_delta_kernel<ElemBF16, 128, false><<<(unsigned)((total_q * p.Hq + 15) / 16), 256, 0, stream>>>(p, total_q);
  {
    static DeviceOnce once;
    const int dev = once.slot();
    if (once.need(dev)) {
      if (hipFuncSetAttribute((const void*)attn_bwd_dq_lds_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, BWL_LDS) != hipSuccess ||
          hipFuncSetAttribute((const void*)attn_bwd_dkv_lds_kernel<BWK_WAVES>, hipFuncAttributeMaxDynamicSharedMemorySize, BWK_LDS) != hipSuccess) {
        (void)hipGetLastError();
        return VX_ERR_LAUNCH;
      }
      once.mark(dev);
    }
  }
  attn_bwd_dq_lds_kernel<<<dim3((unsigned)p.Hq, (unsigned)((max_q + 16 * BWL_WAVES - 1) / (16 * BWL_WAVES)), (unsigned)num_seqs),
                           64 * BWL_WAVES, BWL_LDS, stream>>>(p);
  const int sg = std::max(1, std::min(num_seqs, 8 / std::max(1, p.Hkv)));  // sequences per group of eight workgroups
  attn_bwd_dkv_lds_kernel<BWK_WAVES><<<dim3((unsigned)(p.Hkv * sg), (unsigned)((max_k + 16 * BWK_WAVES - 1) / (16 * BWK_WAVES)),
                                            (unsigned)((num_seqs + sg - 1) / sg)),
                                       64 * BWK_WAVES, BWK_LDS, stream>>>(p);
  return launch_status();
}

}  // namespace vx

extern "C" {

int64_t vx_attention_bwd_workspace_bytes(int64_t total_q, int64_t Hq) { return total_q * Hq * 4; }

// strides[16]: token and head strides (elements) of q, k, v, out, dout, dq, dk, dv, in that order.
int vx_attention_bwd_typed(const void* q, const void* k, const void* v, const void* out, const void* dout, const float* lse,
                           void* dq, void* dk, void* dv, const int* cu_seqlens_q, const int* cu_seqlens_k,
                           int64_t total_q, int64_t total_k, int64_t num_seqs, int Hq, int Hkv, int Dk, int Dv,
                           const int64_t* strides, float softmax_scale, int max_seqlen_q, int max_seqlen_k, int dtype,
                           void* workspace, int64_t workspace_bytes, hipStream_t stream);

int vx_attention_bwd(const void* q, const void* k, const void* v, const void* out, const void* dout, const float* lse,
                     void* dq, void* dk, void* dv, const int* cu_seqlens_q, const int* cu_seqlens_k,
                     int64_t total_q, int64_t total_k, int64_t num_seqs, int Hq, int Hkv, int D,
                     const int64_t* strides, float softmax_scale, int max_seqlen_q, int max_seqlen_k,
                     void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  return vx_attention_bwd_typed(q, k, v, out, dout, lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k, total_q, total_k, num_seqs, Hq,
                                Hkv, D, D, strides, softmax_scale, max_seqlen_q, max_seqlen_k, 0, workspace, workspace_bytes, stream);
}

// Any head sizes up to 256 (Dk of q / k / dq / dk, Dv of v / out / dout / dv) and either 16-bit element type
// (dtype 0 = bf16, 1 = fp16) or fp32 (dtype 2: one thread per gradient row). bf16 at Dk = Dv = 128 runs the LDS kernels, everything else the register-form kernels
// of the next built-for size (64, 128, 256), per element when rows are not 16-byte addressable.
int vx_attention_bwd_typed(const void* q, const void* k, const void* v, const void* out, const void* dout, const float* lse,
                           void* dq, void* dk, void* dv, const int* cu_seqlens_q, const int* cu_seqlens_k,
                           int64_t total_q, int64_t total_k, int64_t num_seqs, int Hq, int Hkv, int Dk, int Dv,
                           const int64_t* strides, float softmax_scale, int max_seqlen_q, int max_seqlen_k, int dtype,
                           void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  using namespace vx;
  if (!q || !k || !v || !out || !dout || !lse || !dq || !dk || !dv || !cu_seqlens_q || !cu_seqlens_k || !strides)
    return VX_ERR_ARG;
  if (total_q < 0 || total_k < 0 || num_seqs < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || Dk <= 0 || Dv <= 0) return VX_ERR_ARG;
  if (max_seqlen_q < 0 || max_seqlen_k < 0 || num_seqs > 65535 || Hq > 65535) return VX_ERR_ARG;
  if (dtype != 0 && dtype != 1 && dtype != 2) return VX_ERR_UNSUPPORTED;
  if (Dk > 256 || Dv > 256) return VX_ERR_UNSUPPORTED;
  if (total_q == 0 || total_k == 0 || num_seqs == 0 || max_seqlen_q == 0 || max_seqlen_k == 0) return VX_OK;
  if (dtype == 2) {  // fp32: one thread per gradient row (attn_f32.h)
    const uintptr_t all = (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)dout | (uintptr_t)dq |
                          (uintptr_t)dk | (uintptr_t)dv | (uintptr_t)workspace;
    if (all % 4 != 0) return VX_ERR_ARG;
    if (!workspace || workspace_bytes < total_q * Hq * 4) return VX_ERR_WORKSPACE;
    AttnF32Bwd f = {};
    f.q = (const float*)q; f.k = (const float*)k; f.v = (const float*)v; f.o = (const float*)out;
    f.d_o = (const float*)dout; f.lse = lse; f.delta = (float*)workspace;
    f.dq = (float*)dq; f.dk = (float*)dk; f.dv = (float*)dv;
    f.sqt = strides[0]; f.sqh = strides[1]; f.skt = strides[2]; f.skh = strides[3];
    f.svt = strides[4]; f.svh = strides[5]; f.sot = strides[6]; f.soh = strides[7];
    f.sdt = strides[8]; f.sdh = strides[9]; f.sdqt = strides[10]; f.sdqh = strides[11];
    f.sdkt = strides[12]; f.sdkh = strides[13]; f.sdvt = strides[14]; f.sdvh = strides[15];
    f.cu_q = cu_seqlens_q; f.cu_k = cu_seqlens_k;
    f.Hq = Hq; f.Hkv = Hkv; f.num_seqs = (int)num_seqs; f.dk_ = Dk; f.dv_ = Dv; f.scale = softmax_scale;
    return launch_attn_f32_backward(f, total_q, total_k, stream);
  }
  const uintptr_t ptrs = (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)dout | (uintptr_t)dq |
                         (uintptr_t)dk | (uintptr_t)dv;
  if (ptrs % 2 != 0) return VX_ERR_ARG;
  bool elem = ptrs % 16 != 0 || Dk % 8 != 0 || Dv % 8 != 0;
  for (int i = 0; i < 16; i++) elem = elem || strides[i] % 8 != 0;
  if (!workspace || workspace_bytes < total_q * Hq * 4 || ((uintptr_t)workspace & 15)) return VX_ERR_WORKSPACE;
  if (total_q * Hq > 0x7fffffffLL * 16) return VX_ERR_ARG;
  AttnBwdParams p = {};
  p.q = (const bf16_t*)q; p.k = (const bf16_t*)k; p.v = (const bf16_t*)v; p.o = (const bf16_t*)out;
  p.d_o = (const bf16_t*)dout; p.lse = lse; p.delta = (float*)workspace;
  p.dq = (bf16_t*)dq; p.dk = (bf16_t*)dk; p.dv = (bf16_t*)dv;
  p.sqt = strides[0]; p.sqh = strides[1]; p.skt = strides[2]; p.skh = strides[3];
  p.svt = strides[4]; p.svh = strides[5]; p.sot = strides[6]; p.soh = strides[7];
  p.sdt = strides[8]; p.sdh = strides[9]; p.sdqt = strides[10]; p.sdqh = strides[11];
  p.sdkt = strides[12]; p.sdkh = strides[13]; p.sdvt = strides[14]; p.sdvh = strides[15];
  p.cu_q = cu_seqlens_q; p.cu_k = cu_seqlens_k;
  p.Hq = Hq; p.Hkv = Hkv; p.num_seqs = (int)num_seqs; p.scale = softmax_scale;
  p.dk_ = Dk; p.dv_ = Dv; p.elem = elem ? 1 : 0;
  const int ns = (int)num_seqs;
  if (dtype == 0 && !elem && Dk == Dv) {
    if (Dk == 128) return launch_attn_bwd_lds128(p, total_q, ns, max_seqlen_q, max_seqlen_k, stream);
    if (Dk == 64) return launch_attn_bwd_generic<ElemBF16, 64, false>(p, total_q, ns, max_seqlen_q, max_seqlen_k, stream);
  }
  const int Db = std::max(Dk, Dv) <= 64 ? 64 : std::max(Dk, Dv) <= 128 ? 128 : 256;
  if (dtype == 1) return launch_attn_bwd_f16(p, Db, total_q, ns, max_seqlen_q, max_seqlen_k, stream);
  if (Db == 64) return launch_attn_bwd_generic<ElemBF16, 64, true>(p, total_q, ns, max_seqlen_q, max_seqlen_k, stream);
  if (Db == 128) return launch_attn_bwd_generic<ElemBF16, 128, true>(p, total_q, ns, max_seqlen_q, max_seqlen_k, stream);
  return launch_attn_bwd_generic<ElemBF16, 256, true>(p, total_q, ns, max_seqlen_q, max_seqlen_k, stream);
}

}  // extern "C"
