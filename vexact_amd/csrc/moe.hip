// Fused MoE block: router top-k, routing integers (histogram, stable expert-major ranks, tile
// table), grouped expert GEMMs and the slot-ordered combine.
// Replaces, for the forward pass:
//   router            vexact/models/qwen3_moe/modeling_qwen3_moe.py:128-134
//   expert_histogram  vexact/batch_invariant_ops/group_gemm/kernel/moe.py:26-81
//   argsort().argsort() ranks / _build_moe_indices   vexact/batch_invariant_ops/fused_moe.py:43, 268-292
//   moe_scatter / moe_gather                          group_gemm/kernel/moe.py:84-161, 253-335
//   group_gemm_same_nk                                group_gemm/kernel/group_gemm.py:65-237
//   silu * up * routing-weight glue                   fused_moe.py:75-88
#include "gemm_core.h"
#include "gemm_wide.h"

namespace vx {

// ---------------------------------------------------------------------------------------
// Router: softmax over E experts in fp32, top-k (ties: lower expert index first), optional
// renormalisation, cast. One wavefront per token, lane owns experts lane, lane+64, ...
// ---------------------------------------------------------------------------------------
constexpr int RT_PER = 8;  // E <= 512

template <bool LOGITS_BF16, bool OUT_BF16, bool IDX64>
__global__ __launch_bounds__(256) void router_topk_kernel(const void* __restrict__ logits,
                                                          void* __restrict__ weights_out,
                                                          void* __restrict__ idx_out, int64_t T,
                                                          int E, int k, int64_t ld, int renorm) {
  const int64_t tok = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tok >= T) return;
  const int lane = threadIdx.x & 63;
  float x[RT_PER];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < RT_PER; i++) {
    const int e = lane + 64 * i;
    if (e < E) {
      if constexpr (LOGITS_BF16) x[i] = bf16_to_f32(((const bf16_t*)logits)[tok * ld + e]);
      else x[i] = ((const float*)logits)[tok * ld + e];
    } else {
      x[i] = -INFINITY;
    }
    mx = fmaxf(mx, x[i]);
  }
  mx = wave_max(mx);
  float pr[RT_PER];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < RT_PER; i++) {
    pr[i] = (lane + 64 * i < E) ? expf(x[i] - mx) : 0.f;
    s += pr[i];
  }
  s = wave_sum(s);
  // k rounds of wave-wide argmax on the logits (same order as on the probabilities)
  float wsel = 0.f;   // lane j < k keeps the j-th selected probability
  int isel = 0;
  float tot = 0.f;
  for (int j = 0; j < k; j++) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    float bp = 0.f;
#pragma unroll
    for (int i = 0; i < RT_PER; i++) {
      const int e = lane + 64 * i;
      if (e < E && (x[i] > bv || (x[i] == bv && e < bi))) { bv = x[i]; bi = e; bp = pr[i]; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      const float op = __shfl_xor(bp, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; bp = op; }
    }
    // retire the winner
#pragma unroll
    for (int i = 0; i < RT_PER; i++)
      if (lane + 64 * i == bi) x[i] = -INFINITY;
    const float p = bp / s;
    tot += p;
    // a row of NaNs wins no comparison: it still gets an expert index inside the table
    if (lane == j) { wsel = p; isel = min(bi, E - 1); }
  }
  if (lane < k) {
    const float w = renorm ? wsel / tot : wsel;
    if constexpr (OUT_BF16) ((bf16_t*)weights_out)[tok * k + lane] = f32_to_bf16(w);
    else ((float*)weights_out)[tok * k + lane] = w;
    if constexpr (IDX64) ((int64_t*)idx_out)[tok * k + lane] = isel;
    else ((int*)idx_out)[tok * k + lane] = isel;
  }
}

// bf16 logits: value and expert index fit one 32-bit key (order-preserving 16 bits of the value above
// 0xffff - e), so a round of the selection is one integer max over the wavefront, done with DPP row
// operations and four lane reads instead of 18 cross-lane permutes. Same selections, same tie rule
// (equal values: lower index; -0 and +0 are equal), and the selected probability is recomputed from
// the winner's value with the expression its owner used, so the outputs are bit-identical to the
// kernel above.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, false));   // lanes i ^ 1
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, false));   // lanes i ^ 2
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, false));  // half-row mirror
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xf, 0xf, false));  // row mirror
  const uint32_t a = __builtin_amdgcn_readlane((int)v, 0), b = __builtin_amdgcn_readlane((int)v, 16);
  const uint32_t c = __builtin_amdgcn_readlane((int)v, 32), d = __builtin_amdgcn_readlane((int)v, 48);
  return max(max(a, b), max(c, d));
}

template <int PER, bool OUT_BF16, bool IDX64>
__global__ __launch_bounds__(256) void router_topk_bf16_kernel(const bf16_t* __restrict__ logits,
                                                               void* __restrict__ weights_out,
                                                               void* __restrict__ idx_out, int64_t T,
                                                               int E, int k, int64_t ld, int renorm) {
  const int64_t tok = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tok >= T) return;
  const int lane = threadIdx.x & 63;
  float x[PER];
  uint32_t key[PER];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const int e = lane + 64 * i;
    key[i] = 0;  // below every real key
    x[i] = -INFINITY;
    if (e < E) {
      uint32_t b = logits[tok * ld + e];
      x[i] = bf16_to_f32((bf16_t)b);
      if (b == 0x8000u) b = 0;  // -0 ties with +0
      const uint32_t ord = (b & 0x8000u) ? (~b & 0xffffu) : (b | 0x8000u);
      key[i] = (ord << 16) | (0xffffu - (uint32_t)e);
    }
    mx = fmaxf(mx, x[i]);
  }
  mx = wave_max(mx);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < PER; i++) s += (lane + 64 * i < E) ? expf(x[i] - mx) : 0.f;
  s = wave_sum(s);
  float wsel = 0.f;
  int isel = 0;
  float tot = 0.f;
  for (int j = 0; j < k; j++) {
    uint32_t best = key[0];
#pragma unroll
    for (int i = 1; i < PER; i++) best = max(best, key[i]);
    best = wave_max_u32(best);
    const int bi = (int)(0xffffu - (best & 0xffffu));
    const uint32_t ord = best >> 16;
    const uint32_t bits = (ord & 0x8000u) ? (ord & 0x7fffu) : (~ord & 0xffffu);
    const float p = expf(bf16_to_f32((bf16_t)bits) - mx) / s;
#pragma unroll
    for (int i = 0; i < PER; i++)
      if (key[i] == best) key[i] = 0;
    tot += p;
    if (lane == j) { wsel = p; isel = bi; }
  }
  if (lane < k) {
    const float w = renorm ? wsel / tot : wsel;
    if constexpr (OUT_BF16) ((bf16_t*)weights_out)[tok * k + lane] = f32_to_bf16(w);
    else ((float*)weights_out)[tok * k + lane] = w;
    if constexpr (IDX64) ((int64_t*)idx_out)[tok * k + lane] = isel;
    else ((int*)idx_out)[tok * k + lane] = isel;
  }
}

// ---------------------------------------------------------------------------------------
// Routing integers, one 1024-thread block. For n = T*k flat entries (token-major, slot-minor):
//   splits[e]         = number of entries routed to expert e
//   cu[e]             = exclusive prefix of splits (cu[E] = n)
//   scatter_index[f]  = position of flat entry f in the stable expert-major order
//   sorted_flat[p]    = f at position p ; sorted_token[p] = f / k
//   tile table        = for each expert, ceil(splits/bm) row tiles of at most bm rows
// All integer, order-independent or explicitly ordered: results are exact.
// ---------------------------------------------------------------------------------------
constexpr int RB_THREADS = 1024;

template <bool IDX64>
__device__ __forceinline__ int route_expert_of(const void* idx, int64_t f, int E) {
  int e;
  if constexpr (IDX64) e = (int)((const int64_t*)idx)[f];
  else e = ((const int*)idx)[f];
  return min(max(e, 0), E - 1);  // keeps later address arithmetic in range
}

// From the per-expert counts in hist (LDS): splits, cu, running[e] = cu[e], first tile of each expert,
// and the tile table. Called by a whole 1024-thread block; ends with the results visible to the block.
__device__ __forceinline__ void route_scan_and_tiles(const int* hist, int* running, int* tstart, int E, int bm,
                                                     int* splits, int* cu, int* tile_group, int* tile_row0,
                                                     int* tile_rows, int max_tiles) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // exclusive scans by wave 0: lane owns experts [lane*per, lane*per+per)
  if (wave == 0) {
    const int per = (E + 63) / 64;
    int c = 0, tl = 0;
    for (int i = 0; i < per; i++) {
      const int e = lane * per + i;
      if (e < E) { c += hist[e]; tl += (hist[e] + bm - 1) / bm; }
    }
    int ci = c, ti = tl;  // inclusive scans across lanes
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int a = __shfl_up(ci, o, 64), b = __shfl_up(ti, o, 64);
      if (lane >= o) { ci += a; ti += b; }
    }
    int cbase = ci - c, tbase = ti - tl;
    for (int i = 0; i < per; i++) {
      const int e = lane * per + i;
      if (e < E) {
        running[e] = cbase;
        tstart[e] = tbase;
        splits[e] = hist[e];
        cu[e] = cbase;
        cbase += hist[e];
        tbase += (hist[e] + bm - 1) / bm;
      }
    }
    if (lane == 63) cu[E] = ci;
  }
  __syncthreads();
  for (int e = tid; e < E; e += RB_THREADS) {
    const int cnt = hist[e], r0 = running[e];
    int t = tstart[e];
    for (int off = 0; off < cnt; off += bm, t++) {
      if (t < max_tiles) {
        tile_group[t] = e;
        tile_row0[t] = r0 + off;
        tile_rows[t] = min(bm, cnt - off);
      }
    }
  }
}

// Stable ranks of the (at most 1024) entries [base, base + 1024) given running[e] = position of the
// next entry of expert e; advances running. wavecnt is [16][E] of LDS. Called by a whole block.
template <bool IDX64>
__device__ __forceinline__ void route_rank_chunk(const void* idx, int64_t base, int64_t n, int k, int E, int ebits,
                                                 int* running, int* wavecnt, int* scatter_index, int* sorted_token,
                                                 int* sorted_flat) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < 16 * E; i += RB_THREADS) wavecnt[i] = 0;
  __syncthreads();
  const int64_t f = base + tid;
  const bool live = f < n;
  const int e = live ? route_expert_of<IDX64>(idx, f, E) : 0;
  // lanes of this wave with the same expert
  uint64_t same = __ballot(live);
  for (int b = 0; b < ebits; b++) {
    const uint64_t bal = __ballot((e >> b) & 1);
    same &= ((e >> b) & 1) ? bal : ~bal;
  }
  if (!live) same = 0;
  const int rank_in_wave = __popcll(same & ((1ull << lane) - 1ull));
  if (live && rank_in_wave == 0) wavecnt[wave * E + e] = __popcll(same);
  __syncthreads();
  for (int ee = tid; ee < E; ee += RB_THREADS) {
    int r = running[ee];
    for (int w = 0; w < 16; w++) {
      const int c = wavecnt[w * E + ee];
      wavecnt[w * E + ee] = r;
      r += c;
    }
    running[ee] = r;
  }
  __syncthreads();
  if (live) {
    const int pos = wavecnt[wave * E + e] + rank_in_wave;
    scatter_index[f] = pos;
    sorted_flat[pos] = (int)f;
    sorted_token[pos] = (int)(f / k);
  }
  __syncthreads();
}

template <bool IDX64>
__global__ __launch_bounds__(RB_THREADS) void moe_route_kernel(
    const void* __restrict__ idx, int64_t n, int k, int E, int bm, int* __restrict__ splits,
    int* __restrict__ cu, int* __restrict__ scatter_index, int* __restrict__ sorted_token,
    int* __restrict__ sorted_flat, int* __restrict__ tile_group, int* __restrict__ tile_row0,
    int* __restrict__ tile_rows, int max_tiles) {
  extern __shared__ int sm[];
  int* hist = sm;             // [E]
  int* running = sm + E;      // [E]  next free position per expert
  int* tstart = sm + 2 * E;   // [E]  first tile of expert
  int* wavecnt = sm + 3 * E;  // [16][E]
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += RB_THREADS) hist[e] = 0;
  for (int t = tid; t < max_tiles; t += RB_THREADS) { tile_group[t] = -1; tile_row0[t] = 0; tile_rows[t] = 0; }
  __syncthreads();
  for (int64_t f = tid; f < n; f += RB_THREADS) atomicAdd(&hist[route_expert_of<IDX64>(idx, f, E)], 1);
  __syncthreads();
  route_scan_and_tiles(hist, running, tstart, E, bm, splits, cu, tile_group, tile_row0, tile_rows, max_tiles);
  int ebits = 0;
  while ((1 << ebits) < E) ebits++;
  for (int64_t base = 0; base < n; base += RB_THREADS)
    route_rank_chunk<IDX64>(idx, base, n, k, E, ebits, running, wavecnt, scatter_index, sorted_token, sorted_flat);
}

// ---- the same routing integers for many entries (prefill): three launches over chunks of 1024 entries.
// counts [chunks][E] (global): first the chunk's expert counts, then (after the scan) the position of the
// chunk's first entry of each expert.
template <bool IDX64>
__global__ __launch_bounds__(RB_THREADS) void moe_route_count_kernel(const void* __restrict__ idx, int64_t n, int E,
                                                                     int* __restrict__ counts) {
  extern __shared__ int sm[];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += RB_THREADS) sm[e] = 0;
  __syncthreads();
  const int64_t f = (int64_t)blockIdx.x * RB_THREADS + tid;
  if (f < n) atomicAdd(&sm[route_expert_of<IDX64>(idx, f, E)], 1);
  __syncthreads();
  for (int e = tid; e < E; e += RB_THREADS) counts[(int64_t)blockIdx.x * E + e] = sm[e];
}

__global__ __launch_bounds__(RB_THREADS) void moe_route_scan_kernel(int* __restrict__ counts, int chunks, int E, int bm,
                                                                    int* __restrict__ splits, int* __restrict__ cu,
                                                                    int* __restrict__ tile_group, int* __restrict__ tile_row0,
                                                                    int* __restrict__ tile_rows, int max_tiles) {
  extern __shared__ int sm[];
  int* hist = sm;
  int* running = sm + E;
  int* tstart = sm + 2 * E;
  const int tid = threadIdx.x;
  for (int t = tid; t < max_tiles; t += RB_THREADS) { tile_group[t] = -1; tile_row0[t] = 0; tile_rows[t] = 0; }
  for (int e = tid; e < E; e += RB_THREADS) {
    int tot = 0;
    for (int c = 0; c < chunks; c++) tot += counts[(int64_t)c * E + e];
    hist[e] = tot;
  }
  __syncthreads();
  route_scan_and_tiles(hist, running, tstart, E, bm, splits, cu, tile_group, tile_row0, tile_rows, max_tiles);
  __syncthreads();
  for (int e = tid; e < E; e += RB_THREADS) {  // counts -> first position of the chunk's entries of expert e
    int base = running[e];
    for (int c = 0; c < chunks; c++) {
      const int t = counts[(int64_t)c * E + e];
      counts[(int64_t)c * E + e] = base;
      base += t;
    }
  }
}

template <bool IDX64>
__global__ __launch_bounds__(RB_THREADS) void moe_route_rank_kernel(const void* __restrict__ idx, int64_t n, int k, int E,
                                                                    const int* __restrict__ counts,
                                                                    int* __restrict__ scatter_index,
                                                                    int* __restrict__ sorted_token,
                                                                    int* __restrict__ sorted_flat) {
  extern __shared__ int sm[];
  int* running = sm;       // [E]
  int* wavecnt = sm + E;   // [16][E]
  for (int e = threadIdx.x; e < E; e += RB_THREADS) running[e] = counts[(int64_t)blockIdx.x * E + e];
  int ebits = 0;
  while ((1 << ebits) < E) ebits++;
  __syncthreads();
  route_rank_chunk<IDX64>(idx, (int64_t)blockIdx.x * RB_THREADS, n, k, E, ebits, running, wavecnt, scatter_index,
                          sorted_token, sorted_flat);
}

template <bool IDX64>
__global__ __launch_bounds__(256) void expert_histogram_kernel(const void* __restrict__ idx, int64_t n,
                                                               int E, int* __restrict__ out) {
  const int64_t f = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (f >= n) return;
  int64_t e;
  if constexpr (IDX64) e = ((const int64_t*)idx)[f];
  else e = ((const int*)idx)[f];
  if (e >= 0 && e < E) atomicAdd(&out[e], 1);
}

__global__ __launch_bounds__(256) void zero_i32_kernel(int* p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0;
}

// out[index[t, i], :] = x[t, :]; one wavefront per (t, i)
__global__ __launch_bounds__(256) void moe_scatter_kernel(const bf16_t* __restrict__ x,
                                                          bf16_t* __restrict__ out,
                                                          const int* __restrict__ index, int64_t n,
                                                          int k, int H, int64_t ldx, int64_t ldo) {
  const int64_t f = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (f >= n) return;
  const int lane = threadIdx.x & 63;
  const bf16_t* src = x + (f / k) * ldx;
  bf16_t* dst = out + (int64_t)index[f] * ldo;
  for (int c = lane; c < H; c += 64) dst[c] = src[c];
}

// y[t, :] = r16( sum_{i<k, ascending} f32(x[index[t, i], :]) ); optional residual:
// y = r16(f32(res[t]) + f32(r16(sum))). One 256-thread block per token. Scalar fallback for
// layouts the vector kernel cannot take.
__global__ __launch_bounds__(256) void moe_gather_kernel(const bf16_t* __restrict__ x,
                                                         const int* __restrict__ index,
                                                         const bf16_t* res, bf16_t* y, int k, int H,
                                                         int64_t ldx, int64_t ldr, int64_t ldy) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < H; c += 256) {
    float acc = 0.f;
    for (int i = 0; i < k; i++) acc += bf16_to_f32(x[(int64_t)index[t * k + i] * ldx + c]);
    bf16_t o = f32_to_bf16(acc);
    if (res) o = f32_to_bf16(bf16_to_f32(res[t * ldr + c]) + bf16_to_f32(o));
    y[t * ldy + c] = o;
  }
}

// Vector version (H % 4 == 0, 8-byte aligned rows) with an optional fused RMSNorm of the result:
// h[t] = rmsnorm(y[t]) with weight nw (mode 1: round(nw * round(y * inv)); mode 0: round(y * inv * nw)).
// Thread t owns the 4-element vectors t, t + 256, ... : the same ownership, in-thread order and
// block reduction as the 256-thread RMSNorm kernel, so fusing does not change a bit.
template <int MAXV>  // vectors per thread kept in registers (H <= 1024 * MAXV)
__global__ __launch_bounds__(256) void moe_gather_vec_kernel(const bf16_t* __restrict__ x,
                                                             const int* __restrict__ index,
                                                             const bf16_t* res, bf16_t* y, int k, int H,
                                                             int64_t ldx, int64_t ldr, int64_t ldy,
                                                             const bf16_t* __restrict__ nw, bf16_t* h,
                                                             int64_t ldh, float eps, int mode, int T,
                                                             const uint4* __restrict__ pf, int64_t pf16) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  if (t >= T) {
    // Workgroups past the tokens read pf16 16-byte pieces and discard them: this kernel leaves most of
    // the memory system idle, and the weights that the next kernel needs cold arrive in the caches
    // meanwhile. The store below never happens; it keeps the loads alive.
    uint32_t acc = 0;
    const int64_t stride = (int64_t)(gridDim.x - T) * 256;
    for (int64_t i = (t - T) * 256 + tid; i < pf16; i += stride) {
      const uint4 v = pf[i];
      acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9e3779b9u && pf16 < 0) y[0] = 0;
    return;
  }
  float o[MAXV][4];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < MAXV; j++) {
    const int c = 4 * (tid + 256 * j);
    if (c < H) {
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
      // slots are summed in ascending order, eight rows requested at a time so that their loads
      // overlap (a slot past k re-reads the last row and is not added)
      for (int i0 = 0; i0 < k; i0 += 8) {
        uint2 raw[8];
#pragma unroll
        for (int u = 0; u < 8; u++)
          raw[u] = *(const uint2*)(x + (int64_t)index[t * k + min(i0 + u, k - 1)] * ldx + c);
#pragma unroll
        for (int u = 0; u < 8; u++) {
          if (i0 + u < k) {
            a0 += bf16lo(raw[u].x); a1 += bf16hi(raw[u].x); a2 += bf16lo(raw[u].y); a3 += bf16hi(raw[u].y);
          }
        }
      }
      uint2 pk;
      pk.x = pack_bf16x2(a0, a1);
      pk.y = pack_bf16x2(a2, a3);
      if (res) {
        const uint2 rr = *(const uint2*)(res + t * ldr + c);
        pk.x = pack_bf16x2(bf16lo(rr.x) + bf16lo(pk.x), bf16hi(rr.x) + bf16hi(pk.x));
        pk.y = pack_bf16x2(bf16lo(rr.y) + bf16lo(pk.y), bf16hi(rr.y) + bf16hi(pk.y));
      }
      *(uint2*)(y + t * ldy + c) = pk;
      o[j][0] = bf16lo(pk.x); o[j][1] = bf16hi(pk.x); o[j][2] = bf16lo(pk.y); o[j][3] = bf16hi(pk.y);
#pragma unroll
      for (int e = 0; e < 4; e++) ss += o[j][e] * o[j][e];
    }
  }
  if (!h) return;
  const float tot = block_sum<4>(ss, red);
  const float inv = rms_inv(tot / (float)H + eps, mode);
#pragma unroll
  for (int j = 0; j < MAXV; j++) {
    const int c = 4 * (tid + 256 * j);
    if (c < H) {
      const uint2 wr = *(const uint2*)(nw + c);
      const float wf[4] = {bf16lo(wr.x), bf16hi(wr.x), bf16lo(wr.y), bf16hi(wr.y)};
      float r[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if (mode == 0) r[e] = o[j][e] * inv * wf[e];
        else r[e] = wf[e] * bf16_to_f32(f32_to_bf16(o[j][e] * inv));
      }
      uint2 pk;
      pk.x = pack_bf16x2(r[0], r[1]);
      pk.y = pack_bf16x2(r[2], r[3]);
      *(uint2*)(h + t * ldh + c) = pk;
    }
  }
}

}  // namespace vx

using namespace vx;

// Fragment-order copy of [G][N][K] weights for the PACKED streaming kernel.
__global__ __launch_bounds__(256) void pack_weights_kernel(const bf16_t* __restrict__ w, int64_t ldw, int64_t gstride,
                                                           int N, int K, int kch, bf16_t* __restrict__ out,
                                                           int64_t pieces) {
  const int64_t pc = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (pc >= pieces) return;
  const int lane = (int)(pc & 63);
  const int64_t frag = pc >> 6;
  const int c = (int)(frag % kch);
  const int64_t nbg = frag / kch;
  const int nblocks = (N + 15) >> 4;
  const int nb = (int)(nbg % nblocks);
  const int64_t grp = nbg / nblocks;
  const int n = 16 * nb + (lane & 15), k0 = 32 * c + 8 * (lane >> 4);
  bf16_t v[8];
#pragma unroll
  for (int j = 0; j < 8; j++) v[j] = (n < N && k0 + j < K) ? w[grp * gstride + (int64_t)n * ldw + k0 + j] : (bf16_t)0;
  uint4 o;
  o.x = (uint32_t)v[0] | ((uint32_t)v[1] << 16);
  o.y = (uint32_t)v[2] | ((uint32_t)v[3] << 16);
  o.z = (uint32_t)v[4] | ((uint32_t)v[5] << 16);
  o.w = (uint32_t)v[6] | ((uint32_t)v[7] << 16);
  *(uint4*)(out + pc * 8) = o;
}

extern "C" {

int vx_router_topk(const void* logits, void* weights_out, void* idx_out, int64_t T, int E, int k,
                   int64_t ld, int logits_bf16, int out_bf16, int idx_i64, int renorm,
                   hipStream_t stream) {
  if (!logits || !weights_out || !idx_out || T < 0 || E <= 0 || k <= 0) return VX_ERR_ARG;
  if (E > 64 * RT_PER || k > 64 || k > E) return VX_ERR_UNSUPPORTED;
  if (T == 0) return VX_OK;
  const int64_t blocks = (T + 3) / 4;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
#define VX_RT(LB, OB, I64)                                                                   \
  router_topk_kernel<LB, OB, I64><<<(unsigned)blocks, 256, 0, stream>>>(logits, weights_out, \
                                                                        idx_out, T, E, k, ld, renorm)
  if (logits_bf16) {
#define VX_RTB(PERV)                                                                                  \
  do {                                                                                                \
    if (out_bf16 && idx_i64) router_topk_bf16_kernel<PERV, true, true><<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)logits, weights_out, idx_out, T, E, k, ld, renorm); \
    else if (out_bf16) router_topk_bf16_kernel<PERV, true, false><<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)logits, weights_out, idx_out, T, E, k, ld, renorm); \
    else if (idx_i64) router_topk_bf16_kernel<PERV, false, true><<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)logits, weights_out, idx_out, T, E, k, ld, renorm); \
    else router_topk_bf16_kernel<PERV, false, false><<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)logits, weights_out, idx_out, T, E, k, ld, renorm); \
  } while (0)
    if (E <= 128) VX_RTB(2);
    else if (E <= 256) VX_RTB(4);
    else VX_RTB(8);
#undef VX_RTB
    return launch_status();
  }
  const int sel = (logits_bf16 ? 4 : 0) | (out_bf16 ? 2 : 0) | (idx_i64 ? 1 : 0);
  switch (sel) {
    case 0: VX_RT(false, false, false); break;
    case 1: VX_RT(false, false, true); break;
    case 2: VX_RT(false, true, false); break;
    case 3: VX_RT(false, true, true); break;
    case 4: VX_RT(true, false, false); break;
    case 5: VX_RT(true, false, true); break;
    case 6: VX_RT(true, true, false); break;
    default: VX_RT(true, true, true); break;
  }
#undef VX_RT
  return launch_status();
}

// upper bound on row tiles: every expert with rows wastes at most one partial tile
int64_t vx_moe_max_tiles(int64_t n_entries, int E, int bm) {
  if (n_entries <= 0 || E <= 0 || bm <= 0) return 0;
  const int64_t a = n_entries < E ? n_entries : E;
  return a + n_entries / bm;
}

// Entries from which the chunked three-launch routing is used when a workspace is given
constexpr int64_t RB_CHUNKED_FROM = 3072;  // one workgroup / chunked, 128 experts: 2048 entries 7.7 / 9.0 us, 3072 10.0 / 9.4, 4096 12.4 / 10.3, 8192 21.8 / 11.5

int64_t vx_moe_route_workspace_bytes(int64_t n_entries, int E) {
  if (n_entries < RB_CHUNKED_FROM || E <= 0) return 0;
  return (n_entries + RB_THREADS - 1) / RB_THREADS * (int64_t)E * 4;
}

int vx_moe_route_ws(const void* expert_idx, int idx_i64, int64_t T, int k, int E, int bm, int* splits,
                    int* cu, int* scatter_index, int* sorted_token, int* sorted_flat, int* tile_group,
                    int* tile_row0, int* tile_rows, int64_t max_tiles, void* workspace, int64_t workspace_bytes,
                    hipStream_t stream) {
  if (!expert_idx || !splits || !cu || !scatter_index || !sorted_token || !sorted_flat ||
      !tile_group || !tile_row0 || !tile_rows)
    return VX_ERR_ARG;
  if (T < 0 || k <= 0 || E <= 0 || bm <= 0) return VX_ERR_ARG;
  if (E > 512) return VX_ERR_UNSUPPORTED;
  const int64_t n = T * k;
  if (n > 0x7fffffffLL) return VX_ERR_ARG;
  if (max_tiles < vx_moe_max_tiles(n, E, bm) || max_tiles > 0x7fffffffLL) return VX_ERR_WORKSPACE;
  const int64_t need = vx_moe_route_workspace_bytes(n, E);
  if (need > 0 && workspace && workspace_bytes >= need && ((uintptr_t)workspace & 3) == 0) {
    const int64_t chunks = (n + RB_THREADS - 1) / RB_THREADS;
    int* counts = (int*)workspace;
    if (idx_i64) moe_route_count_kernel<true><<<(unsigned)chunks, RB_THREADS, (size_t)E * 4, stream>>>(expert_idx, n, E, counts);
    else moe_route_count_kernel<false><<<(unsigned)chunks, RB_THREADS, (size_t)E * 4, stream>>>(expert_idx, n, E, counts);
    moe_route_scan_kernel<<<1, RB_THREADS, (size_t)3 * E * 4, stream>>>(counts, (int)chunks, E, bm, splits, cu, tile_group,
                                                                       tile_row0, tile_rows, (int)max_tiles);
    const size_t lds = (size_t)(1 + 16) * E * 4;
    if (idx_i64)
      moe_route_rank_kernel<true><<<(unsigned)chunks, RB_THREADS, lds, stream>>>(expert_idx, n, k, E, counts, scatter_index,
                                                                                sorted_token, sorted_flat);
    else
      moe_route_rank_kernel<false><<<(unsigned)chunks, RB_THREADS, lds, stream>>>(expert_idx, n, k, E, counts, scatter_index,
                                                                                 sorted_token, sorted_flat);
    return launch_status();
  }
  const size_t lds = (size_t)(3 + 16) * E * sizeof(int);
  if (idx_i64)
    moe_route_kernel<true><<<1, RB_THREADS, lds, stream>>>(expert_idx, n, k, E, bm, splits, cu,
                                                           scatter_index, sorted_token, sorted_flat,
                                                           tile_group, tile_row0, tile_rows,
                                                           (int)max_tiles);
  else
    moe_route_kernel<false><<<1, RB_THREADS, lds, stream>>>(expert_idx, n, k, E, bm, splits, cu,
                                                            scatter_index, sorted_token, sorted_flat,
                                                            tile_group, tile_row0, tile_rows,
                                                            (int)max_tiles);
  return launch_status();
}

int vx_moe_route(const void* expert_idx, int idx_i64, int64_t T, int k, int E, int bm, int* splits,
                 int* cu, int* scatter_index, int* sorted_token, int* sorted_flat, int* tile_group,
                 int* tile_row0, int* tile_rows, int64_t max_tiles, hipStream_t stream) {
  return vx_moe_route_ws(expert_idx, idx_i64, T, k, E, bm, splits, cu, scatter_index, sorted_token, sorted_flat,
                         tile_group, tile_row0, tile_rows, max_tiles, nullptr, 0, stream);
}

// One-wavefront blocks for the streaming kernel: when 4-wavefront blocks would be few (a step of one to four tokens:
// 8 .. 34 expert tiles) and every wavefront has a long run to stream (K >= 1024), four times the workgroups put a
// weight stream on every CU. Measured at 128 experts / top-8, hidden 2048, gate/up on 16-row tiles: 1 token 23.8 ->
// 18.2 us, 3 tokens 41.9 -> 31.9, 4 tokens 46.5 -> 41.0, level from 6 tokens on; the down projection (K = 768, four
// times the blocks already) is level or slower, and so are 32-row tiles.
static inline bool stream_narrow_launch(int64_t max_tiles, int64_t N, int64_t K) {
  return K >= 1024 && max_tiles * ((N + 63) / 64) < 512;
}

// Grouped GEMM over a tile table: C[rows of tile] = X[row_src[rows]] * W[group]^T.
// epi 0: plain bf16 store. epi 1: SwiGLU with w = gate rows, w2 = up rows, scaled per row by
// row_scale[row_scale_idx[row]].  bm in {16, 32, 64} selects the streaming kernel, 128 the tiled one,
// 256 the wide one (x_rows = rows addressable in x; only that kernel needs it).
int vx_moe_gemm(const void* x, int64_t ldx, const void* w, const void* w2, int64_t ldw,
                int64_t w_gstride, void* c, int64_t ldc, int64_t N, int64_t K, const int* tile_group,
                const int* tile_row0, const int* tile_rows, int64_t max_tiles, int bm,
                const int* row_src, const void* row_scale, const int* row_scale_idx, int epi,
                int64_t x_rows, hipStream_t stream) {
  if (!x || !w || !c || !tile_group || !tile_row0 || !tile_rows) return VX_ERR_ARG;
  if (N <= 0 || K <= 0 || N > 0x7fffffff || K > 0x7fffffff || max_tiles < 0) return VX_ERR_ARG;
  if (epi != EPI_PLAIN && epi != EPI_SWIGLU) return VX_ERR_ARG;
  if (epi == EPI_SWIGLU && (!w2 || !row_scale)) return VX_ERR_ARG;
  if (!gemm_fast_ok(x, w, K, ldx, ldw) || (w_gstride % 8) != 0) return VX_ERR_UNSUPPORTED;
  if (epi == EPI_SWIGLU && ((uintptr_t)w2 % 16) != 0) return VX_ERR_UNSUPPORTED;
  if (max_tiles == 0) return VX_OK;
  if (max_tiles > 65535) return VX_ERR_UNSUPPORTED;
  GemmParams p = {};
  p.x = (const bf16_t*)x; p.ldx = ldx;
  p.w = (const bf16_t*)w; p.w2 = (const bf16_t*)w2; p.ldw = ldw; p.w_gstride = w_gstride;
  p.c = (bf16_t*)c; p.ldc = ldc;
  p.M = 0; p.N = (int)N; p.K = (int)K;
  p.tile_group = tile_group; p.tile_row0 = tile_row0; p.tile_rows = tile_rows;
  p.row_src = row_src;
  p.row_scale = (const bf16_t*)row_scale; p.row_scale_idx = row_scale_idx;
  const unsigned my = (unsigned)max_tiles;
  // U = 8 k-steps in flight per wavefront, 32 KB activation chunks (two of these blocks plus
  // their registers fit a CU; measured marginally ahead of 64 KB chunks and of U = 4)
#define VX_GG(MT)                                                                                  \
  do {                                                                                             \
    const dim3 grid((unsigned)((N + 63) / 64), my);                                                \
    if (epi == EPI_SWIGLU) gemm_stream_kernel<MT, EPI_SWIGLU, true, 8, 2><<<grid, 256, 0, stream>>>(p); \
    else gemm_stream_kernel<MT, EPI_PLAIN, true, 8, 2><<<grid, 256, 0, stream>>>(p);               \
  } while (0)
  // a launch of a few 16-row tiles as one-wavefront blocks of 16 weight rows, 256-element activation chunks
#define VX_GG1(MT)                                                                                 \
  do {                                                                                             \
    const dim3 grid((unsigned)((N + 15) / 16), my);                                                \
    if (epi == EPI_SWIGLU) gemm_stream_kernel<MT, EPI_SWIGLU, true, 8, 8, false, 1><<<grid, 64, 0, stream>>>(p); \
    else gemm_stream_kernel<MT, EPI_PLAIN, true, 8, 8, false, 1><<<grid, 64, 0, stream>>>(p);  \
  } while (0)
  const bool narrow = stream_narrow_launch(max_tiles, N, K);
  switch (bm) {
    case 16: if (narrow) VX_GG1(1); else VX_GG(1); break;
    case 32: VX_GG(2); break;
    case 64: VX_GG(4); break;
    case 128: {
      if (epi == EPI_SWIGLU)
        gemm_tiled_kernel<EPI_SWIGLU, true><<<dim3((unsigned)((N + 63) / 64), my), 256, 0, stream>>>(p);
      else
        gemm_tiled_kernel<EPI_PLAIN, true><<<dim3((unsigned)((N + 127) / 128), my), 256, 0, stream>>>(p);
      break;
    }
    case 256:  // prefill sizes: 256x256 tiles, direct-to-LDS loads (needs K % 64 == 0 and x_rows)
      if (x_rows <= 0 || !gemm_wide_grouped_launch(p, epi, max_tiles, x_rows, stream)) return VX_ERR_UNSUPPORTED;
      break;
    default: return VX_ERR_ARG;
  }
#undef VX_GG
#undef VX_GG1
  return launch_status();
}

// ---- fragment-order ("packed") expert weights for the streaming kernel ----
// out[g][nb][c][lane][8] = W_g[16 nb + lane % 16][32 c + 8 (lane / 16) .. + 8], zero past N and K; nb < ceil(N / 16),
// c < kchunks. One thread per 16-byte piece.
int vx_packed_kchunks(int64_t K) { return (int)((K + 255) / 256 * 8); }

int vx_pack_weights(const void* w, int64_t ldw, int64_t w_gstride, int64_t G, int64_t N, int64_t K, void* out,
                    hipStream_t stream) {
  if (!w || !out || G <= 0 || N <= 0 || K <= 0 || N > 0x7fffffff || K > 0x7fffffff) return VX_ERR_ARG;
  if (ldw < K || ((uintptr_t)out % 16) != 0) return VX_ERR_ARG;
  const int kch = vx_packed_kchunks(K);
  const int64_t pieces = G * ((N + 15) / 16) * kch * 64;
  const int64_t blocks = (pieces + 255) / 256;
  if (blocks > 0x7fffffff) return VX_ERR_UNSUPPORTED;
  pack_weights_kernel<<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)w, ldw, w_gstride, (int)N, (int)K, kch,
                                                            (bf16_t*)out, pieces);
  return launch_status();
}

// vx_moe_gemm on packed weights (bm in {16, 32, 64}: streaming kernel; 256: the 256 x 256 kernel, which needs
// K % 64 == 0 and x_rows as vx_moe_gemm does). w / w2 point at the packed image of the first row of the gate / up
// (or only) projection, which must be a multiple of 16 rows into the packed tensor; w_gstride = elements between
// consecutive experts in the packed tensor.
int vx_moe_gemm_packed(const void* x, int64_t ldx, const void* w, const void* w2, int64_t w_gstride, void* c,
                       int64_t ldc, int64_t N, int64_t K, const int* tile_group, const int* tile_row0,
                       const int* tile_rows, int64_t max_tiles, int bm, const int* row_src, const void* row_scale,
                       const int* row_scale_idx, int epi, int64_t x_rows, hipStream_t stream) {
  if (!x || !w || !c || !tile_group || !tile_row0 || !tile_rows) return VX_ERR_ARG;
  if (N <= 0 || K <= 0 || N > 0x7fffffff || K > 0x7fffffff || max_tiles < 0) return VX_ERR_ARG;
  if (epi != EPI_PLAIN && epi != EPI_SWIGLU) return VX_ERR_ARG;
  if (epi == EPI_SWIGLU && (!w2 || !row_scale)) return VX_ERR_ARG;
  if (bm != 16 && bm != 32 && bm != 64 && bm != 256) return VX_ERR_ARG;
  if (((uintptr_t)x % 16) != 0 || ((uintptr_t)w % 16) != 0 || (ldx % 8) != 0 || (w_gstride % 8) != 0)
    return VX_ERR_UNSUPPORTED;
  if (epi == EPI_SWIGLU && ((uintptr_t)w2 % 16) != 0) return VX_ERR_UNSUPPORTED;
  if (max_tiles == 0) return VX_OK;
  if (max_tiles > 65535) return VX_ERR_UNSUPPORTED;
  GemmParams p = {};
  p.x = (const bf16_t*)x; p.ldx = ldx;
  p.w = (const bf16_t*)w; p.w2 = (const bf16_t*)w2; p.ldw = vx_packed_kchunks(K); p.w_gstride = w_gstride;
  p.c = (bf16_t*)c; p.ldc = ldc;
  p.M = 0; p.N = (int)N; p.K = (int)K;
  p.tile_group = tile_group; p.tile_row0 = tile_row0; p.tile_rows = tile_rows;
  p.row_src = row_src;
  p.row_scale = (const bf16_t*)row_scale; p.row_scale_idx = row_scale_idx;
  if (bm == 256) {
    if (x_rows <= 0 || !gemm_wide_grouped_packed_launch(p, epi, max_tiles, x_rows, stream)) return VX_ERR_UNSUPPORTED;
    return launch_status();
  }
  const dim3 grid((unsigned)((N + 63) / 64), (unsigned)max_tiles);
#define VX_GP(MT)                                                                                            \
  do {                                                                                                       \
    if (epi == EPI_SWIGLU) gemm_stream_kernel<MT, EPI_SWIGLU, true, 8, 2, true><<<grid, 256, 0, stream>>>(p); \
    else gemm_stream_kernel<MT, EPI_PLAIN, true, 8, 2, true><<<grid, 256, 0, stream>>>(p);                    \
  } while (0)
#define VX_GP1(MT)                                                                                           \
  do {                                                                                                       \
    const dim3 grid1((unsigned)((N + 15) / 16), (unsigned)max_tiles);                                        \
    if (epi == EPI_SWIGLU) gemm_stream_kernel<MT, EPI_SWIGLU, true, 8, 8, true, 1><<<grid1, 64, 0, stream>>>(p); \
    else gemm_stream_kernel<MT, EPI_PLAIN, true, 8, 8, true, 1><<<grid1, 64, 0, stream>>>(p);            \
  } while (0)
  const bool narrow = stream_narrow_launch(max_tiles, N, K);
  switch (bm) {
    case 16: if (narrow) VX_GP1(1); else VX_GP(1); break;
    case 32: VX_GP(2); break;
    default: VX_GP(4); break;
  }
#undef VX_GP
#undef VX_GP1
  return launch_status();
}

int vx_expert_histogram(const void* idx, int idx_i64, int64_t n, int E, int* out, hipStream_t stream) {
  if (!idx || !out || n < 0 || E <= 0) return VX_ERR_ARG;
  zero_i32_kernel<<<(unsigned)((E + 255) / 256), 256, 0, stream>>>(out, E);  // no memset node: stays graph-safe
  if (n == 0) return VX_OK;
  const int64_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
  if (idx_i64) expert_histogram_kernel<true><<<(unsigned)blocks, 256, 0, stream>>>(idx, n, E, out);
  else expert_histogram_kernel<false><<<(unsigned)blocks, 256, 0, stream>>>(idx, n, E, out);
  return launch_status();
}

int vx_moe_scatter(const void* x, void* out, const int* index, int64_t T, int k, int64_t H,
                   int64_t ldx, int64_t ldo, hipStream_t stream) {
  if (!x || !out || !index || T < 0 || k <= 0 || H <= 0 || H > 0x7fffffff) return VX_ERR_ARG;
  const int64_t n = T * k;
  if (n == 0) return VX_OK;
  const int64_t blocks = (n + 3) / 4;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
  moe_scatter_kernel<<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, index, n,
                                                           k, (int)H, ldx, ldo);
  return launch_status();
}

// y = gather-sum (+ residual); when norm_weight and h are given, also h = RMSNorm(y) (mode as in
// vx_rms_norm). The fused norm needs H % 4 == 0, H <= 8192 and 8-byte aligned rows.
// prefetch / prefetch_bytes (optional, vector path only): memory that extra workgroups read and discard
// while the combine runs, e.g. the weights of the projection that follows.
int vx_moe_gather_norm_prefetch(const void* x, const int* index, const void* residual, void* y, int64_t T, int k,
                                int64_t H, int64_t ldx, int64_t ldr, int64_t ldy, const void* norm_weight, void* h,
                                int64_t ldh, float eps, int mode, const void* prefetch, int64_t prefetch_bytes,
                                hipStream_t stream) {
  if (!x || !y || !index || T < 0 || k <= 0 || H <= 0 || H > 0x7fffffff) return VX_ERR_ARG;
  if (prefetch_bytes < 0 || (prefetch && ((uintptr_t)prefetch % 16) != 0)) return VX_ERR_ARG;
  if ((norm_weight == nullptr) != (h == nullptr)) return VX_ERR_ARG;
  if (mode != 0 && mode != 1) return VX_ERR_ARG;
  if (T == 0) return VX_OK;
  if (T > 0x7fffffffLL) return VX_ERR_ARG;
  const bool vec = (H % 4 == 0) && (ldx % 4 == 0) && (ldy % 4 == 0) && (ldr % 4 == 0) && (ldh % 4 == 0) &&
                   (((uintptr_t)x | (uintptr_t)y | (uintptr_t)residual | (uintptr_t)h | (uintptr_t)norm_weight) % 8 == 0) &&
                   H <= 8192;
  if (!vec) {
    if (h) return VX_ERR_UNSUPPORTED;
    moe_gather_kernel<<<(unsigned)T, 256, 0, stream>>>((const bf16_t*)x, index, (const bf16_t*)residual,
                                                       (bf16_t*)y, k, (int)H, ldx, ldr, ldy);
    return launch_status();
  }
  const int64_t pf16 = prefetch ? prefetch_bytes / 16 : 0;
  const int64_t pfb = pf16 > 0 ? (pf16 + 1023) / 1024 : 0;  // four pieces per thread, at most 1024 workgroups
  const unsigned grid = (unsigned)(T + (pfb > 1024 ? 1024 : pfb));
#define VX_GV(MV)                                                                                     \
  moe_gather_vec_kernel<MV><<<grid, 256, 0, stream>>>(                                                \
      (const bf16_t*)x, index, (const bf16_t*)residual, (bf16_t*)y, k, (int)H, ldx, ldr, ldy,         \
      (const bf16_t*)norm_weight, (bf16_t*)h, ldh, eps, mode, (int)T, (const uint4*)prefetch, pf16)
  if (H <= 1024) VX_GV(1);
  else if (H <= 2048) VX_GV(2);
  else if (H <= 4096) VX_GV(4);
  else VX_GV(8);
#undef VX_GV
  return launch_status();
}

int vx_moe_gather_norm(const void* x, const int* index, const void* residual, void* y, int64_t T, int k,
                       int64_t H, int64_t ldx, int64_t ldr, int64_t ldy, const void* norm_weight, void* h,
                       int64_t ldh, float eps, int mode, hipStream_t stream) {
  return vx_moe_gather_norm_prefetch(x, index, residual, y, T, k, H, ldx, ldr, ldy, norm_weight, h, ldh, eps, mode,
                                     nullptr, 0, stream);
}

int vx_moe_gather(const void* x, const int* index, const void* residual, void* y, int64_t T, int k,
                  int64_t H, int64_t ldx, int64_t ldr, int64_t ldy, hipStream_t stream) {
  return vx_moe_gather_norm(x, index, residual, y, T, k, H, ldx, ldr, ldy, nullptr, nullptr, 0, 0.f, 1, stream);
}

}  // extern "C"
