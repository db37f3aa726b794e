// Row-wise reductions: mean over one dim, RMSNorm (two rounding variants, optional fused
// residual add), log_softmax, per-token logprob and greedy argmax.
//
// All of them are HBM-bound. One row is always reduced by one fixed-size thread group whose
// size depends on the row length only; a thread owns the 4-element vectors t, t+G, t+2G, ...
// and adds their elements in ascending order, then a lane butterfly and an ascending
// wave-order pass finish the sum. The schedule never looks at the number of rows.
#include <algorithm>

#include "common.h"
#include <math.h>
#include <atomic>

namespace vx {

enum : int { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2 };

template <int DT> struct Elem;
template <> struct Elem<DT_F32> {
  using T = float;
  static __device__ __forceinline__ float ld(const T* p) { return *p; }
  static __device__ __forceinline__ void st(T* p, float v) { *p = v; }
};
template <> struct Elem<DT_BF16> {
  using T = bf16_t;
  static __device__ __forceinline__ float ld(const T* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void st(T* p, float v) { *p = f32_to_bf16(v); }
};
template <> struct Elem<DT_F16> {
  using T = _Float16;
  static __device__ __forceinline__ float ld(const T* p) { return (float)*p; }
  static __device__ __forceinline__ void st(T* p, float v) { *p = (_Float16)v; }
};

// ---------------------------------------------------------------------------------------
// mean over the middle dim of an (M, N, K) strided view.
// Replaces mean_kernel / mean_dim (vexact/batch_invariant_ops/batch_invariant_ops.py:336-473).
// G threads per output element: 64 when N <= 512, else 256.
// ---------------------------------------------------------------------------------------
template <int DT, int G>
__global__ __launch_bounds__(256) void mean_dim_kernel(const typename Elem<DT>::T* __restrict__ in,
                                                       typename Elem<DT>::T* __restrict__ out,
                                                       int64_t s0, int64_t s1, int64_t s2,
                                                       int64_t o0, int64_t o1, int64_t M, int64_t N,
                                                       int64_t K) {
  __shared__ float red[4];
  constexpr int RPB = 256 / G;  // output elements per block
  const int sub = threadIdx.x / G;
  const int t = threadIdx.x % G;
  const int64_t oid = (int64_t)blockIdx.x * RPB + sub;
  const bool live = oid < M * K;
  float acc = 0.f;
  if (live) {
    const int64_t m = oid / K, k = oid % K;
    const typename Elem<DT>::T* base = in + m * s0 + k * s2;
    for (int64_t v = t; v * 4 < N; v += G) {
      const int64_t n0 = v * 4;
#pragma unroll
      for (int c = 0; c < 4; c++)
        if (n0 + c < N) acc += Elem<DT>::ld(base + (n0 + c) * s1);
    }
  }
  float tot;
  if constexpr (G == 64) tot = wave_sum(acc);
  else tot = block_sum<4>(acc, red);
  if (live && t == 0) {
    const int64_t m = oid / K, k = oid % K;
    Elem<DT>::st(out + m * o0 + k * o1, tot / (float)N);
  }
}

// ---------------------------------------------------------------------------------------
// RMSNorm over the last dim of [rows, n].
// mode 0: y = r16(f32(x) * inv * f32(w)), inv = 1/sqrt(ss/n + eps)  -- one rounding;
//         replaces _rms_norm_kernel (batch_invariant_ops.py:637-669).
// mode 1: y = r16(f32(w) * f32(r16(f32(x) * inv)))                  -- the two-rounding form a
//         HuggingFace Qwen3 RMSNorm produces when its .mean(-1) runs through mean_dim.
// If res != nullptr the row is first replaced by r16(x + res) (a bf16 residual add) and that
// sum is also written to sum_out.
// ---------------------------------------------------------------------------------------
template <int DT, int G>
__global__ __launch_bounds__(256) void rms_norm_kernel(
    const typename Elem<DT>::T* x, const typename Elem<DT>::T* res,
    const typename Elem<DT>::T* __restrict__ w, typename Elem<DT>::T* y,
    typename Elem<DT>::T* sum_out, int64_t rows, int n, int64_t xs, int64_t rs,
    int64_t ys, int64_t ss, float eps, int mode) {
  using E = Elem<DT>;
  __shared__ float red[4];
  constexpr int RPB = 256 / G;
  const int sub = threadIdx.x / G;
  const int t = threadIdx.x % G;
  const int64_t row = (int64_t)blockIdx.x * RPB + sub;
  const bool live = row < rows;
  const typename E::T* xr = x + row * xs;
  const typename E::T* rr = res ? res + row * rs : nullptr;
  typename E::T* so = sum_out ? sum_out + row * ss : nullptr;
  float acc = 0.f;
  if (live) {
    for (int v = t; v * 4 < n; v += G) {
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int j = v * 4 + c;
        if (j < n) {
          float f = E::ld(xr + j);
          if (rr) {
            // round the residual sum to the storage type before it is used
            typename E::T tmp;
            E::st(&tmp, f + E::ld(rr + j));
            f = E::ld(&tmp);
            if (so) so[j] = tmp;
          }
          acc += f * f;
        }
      }
    }
  }
  float tot;
  if constexpr (G == 64) tot = wave_sum(acc);
  else tot = block_sum<4>(acc, red);
  if (!live) return;
  const float inv = rms_inv(tot / (float)n + eps, mode);
  typename E::T* yr = y + row * ys;
  for (int v = t; v * 4 < n; v += G) {
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const int j = v * 4 + c;
      if (j < n) {
        float f;
        if (rr && so) {
          f = E::ld(so + j);  // written by this thread above; safe when sum_out aliases x or res
        } else {
          f = E::ld(xr + j);
          if (rr) {
            typename E::T tmp;
            E::st(&tmp, f + E::ld(rr + j));
            f = E::ld(&tmp);
          }
        }
        const float wf = E::ld(w + j);
        if (mode == 0) {
          E::st(yr + j, f * inv * wf);
        } else {
          typename E::T tmp;
          E::st(&tmp, f * inv);
          E::st(yr + j, wf * E::ld(&tmp));
        }
      }
    }
  }
}

// bf16 fast path of rms_norm_kernel: 8-byte loads/stores, row values kept in registers. Same
// element ownership, in-thread order and reductions as the generic kernel, hence the same bits.
// Requirements (checked by the launcher): n % 4 == 0, n <= 1024 * MAXV (G = 256) or n <= 512
// (G = 64), strides % 4 == 0, 8-byte aligned pointers.
template <int G, int MAXV>
__global__ __launch_bounds__(256) void rms_norm_bf16v_kernel(const bf16_t* x, const bf16_t* res,
                                                             const bf16_t* __restrict__ w, bf16_t* y,
                                                             bf16_t* sum_out, int64_t rows, int n,
                                                             int64_t xs, int64_t rs, int64_t ys, int64_t ss,
                                                             float eps, int mode) {
  __shared__ float red[4];
  constexpr int RPB = 256 / G;
  const int sub = threadIdx.x / G, t = threadIdx.x % G;
  const int64_t row = (int64_t)blockIdx.x * RPB + sub;
  const bool live = row < rows;
  float f[MAXV][4];
  float acc = 0.f;
  if (live) {
#pragma unroll
    for (int j = 0; j < MAXV; j++) {
      const int c = 4 * (t + G * j);
      if (c < n) {
        uint2 raw = *(const uint2*)(x + row * xs + c);
        if (res) {
          const uint2 rr = *(const uint2*)(res + row * rs + c);
          raw.x = pack_bf16x2(bf16lo(raw.x) + bf16lo(rr.x), bf16hi(raw.x) + bf16hi(rr.x));
          raw.y = pack_bf16x2(bf16lo(raw.y) + bf16lo(rr.y), bf16hi(raw.y) + bf16hi(rr.y));
          if (sum_out) *(uint2*)(sum_out + row * ss + c) = raw;
        }
        f[j][0] = bf16lo(raw.x); f[j][1] = bf16hi(raw.x); f[j][2] = bf16lo(raw.y); f[j][3] = bf16hi(raw.y);
#pragma unroll
        for (int e = 0; e < 4; e++) acc += f[j][e] * f[j][e];
      }
    }
  }
  float tot;
  if constexpr (G == 64) tot = wave_sum(acc);
  else tot = block_sum<4>(acc, red);
  if (!live) return;
  const float inv = rms_inv(tot / (float)n + eps, mode);
#pragma unroll
  for (int j = 0; j < MAXV; j++) {
    const int c = 4 * (t + G * j);
    if (c < n) {
      const uint2 wr = *(const uint2*)(w + c);
      const float wf[4] = {bf16lo(wr.x), bf16hi(wr.x), bf16lo(wr.y), bf16hi(wr.y)};
      float r[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if (mode == 0) r[e] = f[j][e] * inv * wf[e];
        else r[e] = wf[e] * bf16_to_f32(f32_to_bf16(f[j][e] * inv));
      }
      uint2 pk;
      pk.x = pack_bf16x2(r[0], r[1]);
      pk.y = pack_bf16x2(r[2], r[3]);
      *(uint2*)(y + row * ys + c) = pk;
    }
  }
}

// ---------------------------------------------------------------------------------------
// log_softmax / logprob / argmax over rows of [rows, n], split into fixed chunks of
// LS_CHUNK columns so that few rows still fill the chip. The chunk count depends on n only.
// Pass 1 writes per (row, chunk): max m_c, s_c = sum exp(x - m_c), and the first index of
// the max. Pass 2 folds the partials in ascending chunk order:
//   m = max_c m_c ; S = sum_c s_c * exp(m_c - m) ; y = (x - m) - log(S).
// Replaces _log_softmax_kernel / log_softmax (batch_invariant_ops.py:231-333) and the
// cross-entropy call behind logprobs_from_logits_flash_attn (standalone_logprobs.py:28-55).
// ---------------------------------------------------------------------------------------
constexpr int LS_CHUNK = 4096;
constexpr int LS_THREADS = 256;
constexpr int LS_PER = LS_CHUNK / LS_THREADS;  // 16 values per thread

struct LsPartial {
  float m;
  float s;
  int idx;
  int pad;
};

// four consecutive elements at p: one 16- or 8-byte access when `vec` (p is aligned to the four elements and all
// four lie inside the row), element by element otherwise; same values either way
template <int DT>
__device__ __forceinline__ void ls_load4(const typename Elem<DT>::T* p, int left, bool vec, float* v) {
  using T = typename Elem<DT>::T;
  if (vec) {
    __attribute__((aligned(16))) T t[4];
    if constexpr (sizeof(T) == 4) *(uint4*)t = *(const uint4*)p;
    else *(uint2*)t = *(const uint2*)p;
#pragma unroll
    for (int c = 0; c < 4; c++) v[c] = Elem<DT>::ld(t + c);
  } else {
#pragma unroll
    for (int c = 0; c < 4; c++) v[c] = (c < left) ? Elem<DT>::ld(p + c) : -INFINITY;
  }
}

template <int DT>
__device__ __forceinline__ void ls_load(const typename Elem<DT>::T* row, int n, int c0, float* v) {
  // thread t owns vectors t, t+256, t+512, t+768 of the chunk (4 elements each)
  const bool aligned = ((uintptr_t)row % (4 * sizeof(typename Elem<DT>::T))) == 0;  // chunk and vector starts are multiples of 4
#pragma unroll
  for (int j = 0; j < LS_PER / 4; j++) {
    const int e0 = c0 + 4 * (threadIdx.x + LS_THREADS * j);
    ls_load4<DT>(row + e0, n - e0, aligned && e0 + 3 < n, v + 4 * j);
  }
}

template <int DT>
__global__ __launch_bounds__(LS_THREADS) void ls_partial_kernel(
    const typename Elem<DT>::T* __restrict__ x, LsPartial* __restrict__ part, int n, int64_t xs,
    int nchunk) {
  __shared__ float red[4];
  __shared__ int redi[4];
  const int64_t row = blockIdx.y;
  const int ch = blockIdx.x;
  const int c0 = ch * LS_CHUNK;
  float v[LS_PER];
  ls_load<DT>(x + row * xs, n, c0, v);
  float m = v[0];
  int mi = 0;
#pragma unroll
  for (int i = 1; i < LS_PER; i++)
    if (v[i] > m) { m = v[i]; mi = i; }
  // element index of this thread's local max
  int idx = c0 + 4 * (threadIdx.x + LS_THREADS * (mi / 4)) + (mi % 4);
  const float bm = block_max<4>(m, red);
  // first index holding the block max
  int cand = (m == bm) ? idx : 0x7fffffff;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, 64));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) redi[threadIdx.x >> 6] = cand;
  __syncthreads();
  cand = min(min(redi[0], redi[1]), min(redi[2], redi[3]));
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < LS_PER; i++) s += (v[i] == -INFINITY) ? 0.f : expf(v[i] - bm);  // padded tail adds 0
  const float bs = block_sum<4>(s, red);
  if (threadIdx.x == 0) {
    LsPartial p;
    p.m = bm; p.s = bs; p.idx = cand; p.pad = 0;
    part[row * nchunk + ch] = p;
  }
}

// Folds a row's chunk partials: m = max_c m_c (amax = index stored with the first chunk that attains it),
// S = sum over ascending c of s_c * exp(m_c - m), logS = log S. One wavefront does it together: lane l takes chunks
// l, l + 64, ... for the maximum and the terms, and the terms are then added one by one in ascending chunk order
// (every lane carries the same running sum), so the result is the sequential sum, bit for bit, at 1/64 of its
// exponentials per lane. All 64 lanes of the calling wavefront must be active.
__device__ __forceinline__ void ls_fold_wave(const LsPartial* __restrict__ p, int nchunk, float& m,
                                             float& logS, int& amax) {
  const int lane = threadIdx.x & 63;
  float bm = -INFINITY;
  int bc = 0x7fffffff;  // first chunk attaining bm among this lane's chunks
  for (int c = lane; c < nchunk; c += 64) {
    const float v = p[c].m;
    if (v > bm || bc == 0x7fffffff) { bm = v; bc = c; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float om = __shfl_xor(bm, o, 64);
    const int oc = __shfl_xor(bc, o, 64);
    if (oc != 0x7fffffff && (bc == 0x7fffffff || om > bm || (om == bm && oc < bc))) { bm = om; bc = oc; }
  }
  m = bm;
  amax = p[bc].idx;
  float S = 0.f;
  for (int base = 0; base < nchunk; base += 64) {
    const int c = base + lane;
    const float t = c < nchunk ? p[c].s * expf(p[c].m - m) : 0.f;
    const int cnt = min(64, nchunk - base);
    for (int i = 0; i < cnt; i++) S += __shfl(t, i, 64);
  }
  logS = logf(S);
}

// CPW = consecutive chunks of a row that one workgroup finishes (the fold of the row's partials is done once per
// workgroup, and CPW chunks of loads are in flight per thread): 1 when the launch has few (row, chunk) pairs, 4
// when it has thousands (fp32, 64 rows x 38 chunks: 18.7 -> 14.8 us; the partial kernel is faster with one chunk per
// workgroup, 9.6 against 11.6 us with two). Which workgroup writes an element changes nothing about its value.
template <int DT, int CPW>
__global__ __launch_bounds__(LS_THREADS) void ls_final_kernel(
    const typename Elem<DT>::T* __restrict__ x, typename Elem<DT>::T* __restrict__ y,
    const LsPartial* __restrict__ part, int n, int64_t xs, int64_t ys, int nchunk) {
  __shared__ float fold[2];
  const int64_t row = blockIdx.y;
  const int c_first = blockIdx.x * (CPW * LS_CHUNK);
  const typename Elem<DT>::T* xr = x + row * xs;
  typename Elem<DT>::T* yr = y + row * ys;
  using T = typename Elem<DT>::T;
  const bool aligned = (((uintptr_t)xr | (uintptr_t)yr) % (4 * sizeof(T))) == 0;
  // the chunks' values are requested first: their way from memory overlaps the fold of the row's partials
  float v[CPW][LS_PER];
  bool vec[CPW][LS_PER / 4];
#pragma unroll
  for (int cc = 0; cc < CPW; cc++)
#pragma unroll
    for (int j = 0; j < LS_PER / 4; j++) {
      const int e0 = c_first + cc * LS_CHUNK + 4 * (threadIdx.x + LS_THREADS * j);
      vec[cc][j] = aligned && e0 + 3 < n;
      if (e0 < n) ls_load4<DT>(xr + e0, n - e0, vec[cc][j], v[cc] + 4 * j);
    }
  if (threadIdx.x < 64) {  // the first wavefront folds the row's partials for the block
    float fm, fl;
    int amax;
    ls_fold_wave(part + row * nchunk, nchunk, fm, fl, amax);
    if (threadIdx.x == 0) { fold[0] = fm; fold[1] = fl; }
  }
  __syncthreads();
  const float m = fold[0], logS = fold[1];
#pragma unroll
  for (int cc = 0; cc < CPW; cc++)
#pragma unroll
    for (int j = 0; j < LS_PER / 4; j++) {
      const int e0 = c_first + cc * LS_CHUNK + 4 * (threadIdx.x + LS_THREADS * j);
      if (e0 >= n) continue;
      if (vec[cc][j]) {
        __attribute__((aligned(16))) T t[4];
#pragma unroll
        for (int c = 0; c < 4; c++) Elem<DT>::st(t + c, (v[cc][4 * j + c] - m) - logS);
        if constexpr (sizeof(T) == 4) *(uint4*)(yr + e0) = *(const uint4*)t;
        else *(uint2*)(yr + e0) = *(const uint2*)t;
      } else {
#pragma unroll
        for (int c = 0; c < 4; c++)
          if (e0 + c < n) Elem<DT>::st(yr + e0 + c, (v[cc][4 * j + c] - m) - logS);
      }
    }
}

// out[row] = (x[row, label] - m) - log S ; when labels == nullptr the greedy token (first
// argmax) is used and also written to tok_out.
template <int DT>
__global__ __launch_bounds__(64) void logprob_final_kernel(
    const typename Elem<DT>::T* __restrict__ x, const int64_t* __restrict__ labels,
    const LsPartial* __restrict__ part, float* __restrict__ out, int64_t* __restrict__ tok_out,
    int64_t rows, int n, int64_t xs, int nchunk) {
  const int64_t row = blockIdx.x;  // one wavefront per row
  float m, logS;
  int amax;
  ls_fold_wave(part + row * nchunk, nchunk, m, logS, amax);
  if (threadIdx.x != 0) return;
  int64_t lab = labels ? labels[row] : (int64_t)amax;
  if (tok_out) tok_out[row] = lab;
  float r = NAN;
  if (lab >= 0 && lab < n) r = (Elem<DT>::ld(x + row * xs + lab) - m) - logS;
  out[row] = r;
}

}  // namespace vx

using namespace vx;

// ---------------------------------------------------------------------------------------
// Chunk partials of vx_logprobs_static live in this array instead of a caller's workspace. The
// name `scratch` is a host-side stand-in for the symbol: host code uses the per-device address
// that hipGetSymbolAddress returns (every GPU holds its own copy at its own address).
// ---------------------------------------------------------------------------------------
constexpr int64_t kStaticScratchBytes = 1 << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device, looked up once per device.
static int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return VX_ERR_LAUNCH;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return VX_ERR_LAUNCH;
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing first calls store the same address
  }
  *out = p;
  return VX_OK;
}

// Backward of RMSNorm y = w r(x inv) (mode 1: h = x inv is rounded to the storage type before the weight is applied,
// as in HuggingFace's forward) or y = r(w x inv) (mode 0), inv = 1 / sqrt(mean(x^2) + eps), for 16-bit storage types:
//   d_h = d_y w,  d_x = inv (d_h - h mean(d_h h)),  d_w = sum over rows of d_y r(h).
// G lanes share a row (8-element pieces, up to MAXV per lane); a workgroup's 256 / G row slots walk the rows with the
// grid's stride and keep d_w sums for their own columns in registers; at the end the slots add them in slot order into
// LDS and the workgroup writes one fp32 partial row. rms_norm_bwd_finish_kernel adds the partial rows in workgroup
// order: run-to-run deterministic for a given number of rows.
template <int DT, int G, int MAXV>
__global__ __launch_bounds__(256) void rms_norm_bwd_kernel(const typename Elem<DT>::T* __restrict__ x,
                                                           const typename Elem<DT>::T* __restrict__ w,
                                                           const typename Elem<DT>::T* __restrict__ dy,
                                                           typename Elem<DT>::T* __restrict__ dx, float* __restrict__ dw_part,
                                                           int64_t rows, int n, int64_t xs, int64_t dys, int64_t dxs,
                                                           float eps, int mode) {
  using E = Elem<DT>;
  using T = typename E::T;
  constexpr int SLOTS = 256 / G;
  extern __shared__ float rb_red[];  // n floats
  const int slot = threadIdx.x / G, l = threadIdx.x % G;
  const int nv = n >> 3;
  auto ld8 = [](const T* p, float (&f)[8]) {
    const uint4 raw = *(const uint4*)p;
    const T* e = (const T*)&raw;
#pragma unroll
    for (int c = 0; c < 8; c++) f[c] = E::ld(e + c);
  };
  float wf[MAXV][8], acc[MAXV][8];
#pragma unroll
  for (int i = 0; i < MAXV; i++) {
    const int v = l + i * G;
#pragma unroll
    for (int c = 0; c < 8; c++) { wf[i][c] = 0.f; acc[i][c] = 0.f; }
    if (v < nv) ld8(w + 8 * v, wf[i]);
  }
  for (int64_t r = (int64_t)blockIdx.x * SLOTS + slot; r < rows; r += (int64_t)gridDim.x * SLOTS) {
    float xf[MAXV][8], gf[MAXV][8];
    float ssq = 0.f;
#pragma unroll
    for (int i = 0; i < MAXV; i++) {
      const int v = l + i * G;
      if (v < nv) {
        ld8(x + r * xs + 8 * v, xf[i]);
        ld8(dy + r * dys + 8 * v, gf[i]);
      } else {
#pragma unroll
        for (int c = 0; c < 8; c++) { xf[i][c] = 0.f; gf[i][c] = 0.f; }
      }
#pragma unroll
      for (int c = 0; c < 8; c++) ssq += xf[i][c] * xf[i][c];
    }
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) ssq += __shfl_xor(ssq, o, 64);
    const float inv = rms_inv(ssq / (float)n + eps, mode);
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < MAXV; i++)
#pragma unroll
      for (int c = 0; c < 8; c++) {
        const float h = xf[i][c] * inv;
        T hb;
        E::st(&hb, h);
        acc[i][c] += gf[i][c] * (mode == 1 ? E::ld(&hb) : h);
        gf[i][c] *= wf[i][c];  // d_h
        xf[i][c] = h;
        dot += gf[i][c] * h;
      }
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) dot += __shfl_xor(dot, o, 64);
    const float cm = dot / (float)n;
#pragma unroll
    for (int i = 0; i < MAXV; i++) {
      const int v = l + i * G;
      if (v < nv) {
        uint4 o4;
        T* e = (T*)&o4;
#pragma unroll
        for (int c = 0; c < 8; c++) E::st(e + c, inv * (gf[i][c] - xf[i][c] * cm));
        *(uint4*)(dx + r * dxs + 8 * v) = o4;
      }
    }
  }
  for (int s = 0; s < SLOTS; s++) {
    if (slot == s) {
#pragma unroll
      for (int i = 0; i < MAXV; i++) {
        const int v = l + i * G;
        if (v < nv) {
#pragma unroll
          for (int c = 0; c < 8; c++) rb_red[8 * v + c] = (s == 0 ? 0.f : rb_red[8 * v + c]) + acc[i][c];
        }
      }
    }
    __syncthreads();
  }
  for (int j = threadIdx.x; j < n; j += 256) dw_part[(int64_t)blockIdx.x * n + j] = rb_red[j];
}

// 64 columns per workgroup; wavefront v of 8 adds the partial rows v, v + 8, ... in ascending order, then the eight sums
// are added in wavefront order
template <int DT>
__global__ __launch_bounds__(512) void rms_norm_bwd_finish_kernel(const float* __restrict__ dw_part, int nblocks, int n,
                                                                  typename Elem<DT>::T* __restrict__ dw) {
  __shared__ float part[8][64];
  const int lane = threadIdx.x & 63, v = threadIdx.x >> 6;
  const int j = blockIdx.x * 64 + lane;
  float s = 0.f;
  if (j < n)
    for (int b = v; b < nblocks; b += 8) s += dw_part[(int64_t)b * n + j];
  part[v][lane] = s;
  __syncthreads();
  if (v == 0 && j < n) {
    float t = part[0][lane];
#pragma unroll
    for (int i = 1; i < 8; i++) t += part[i][lane];
    Elem<DT>::st(dw + j, t);
  }
}

// Gradient of out[i] = logits[i, label_i] - logsumexp(logits[i, :]) with respect to the logits, from the forward's
// output: lse_i = logits[i, label_i] - out[i], d_logits[i, j] = d_out[i] ((j == label_i) - exp(logits[i, j] - lse_i)).
// Elementwise over the row; d_logits may be the logits' own memory (every element is read before it is written).
template <int DT>
__global__ __launch_bounds__(256) void logprob_bwd_kernel(const typename Elem<DT>::T* logits,  // may alias d_logits
                                                          const int64_t* __restrict__ labels,
                                                          const float* __restrict__ out, const float* __restrict__ d_out,
                                                          typename Elem<DT>::T* d_logits, int n, int64_t x_stride,
                                                          int64_t d_stride) {
  const int64_t row = blockIdx.y;
  const int64_t lab = labels[row];
  const typename Elem<DT>::T* x = logits + row * x_stride;
  typename Elem<DT>::T* d = d_logits + row * d_stride;
  const float g = d_out[row];
  const bool has = lab >= 0 && lab < n;
  const float lse = has ? Elem<DT>::ld(x + lab) - out[row] : 0.f;
  __syncthreads();  // in place: everyone has read the label's logit before anyone overwrites it
  for (int j = blockIdx.x * 256 + threadIdx.x; j < n; j += gridDim.x * 256) {
    const float p = has ? expf(Elem<DT>::ld(x + j) - lse) : 0.f;
    Elem<DT>::st(d + j, g * ((j == lab ? 1.f : 0.f) - p));
  }
}

extern "C" {

int vx_mean_dim(const void* in, void* out, int dtype, int64_t M, int64_t N, int64_t K, int64_t s0,
                int64_t s1, int64_t s2, int64_t o0, int64_t o1, hipStream_t stream) {
  if (!in || !out || M < 0 || N <= 0 || K < 0) return VX_ERR_ARG;
  const int64_t outs = M * K;
  if (outs == 0) return VX_OK;
  const bool small = N <= 512;
  const int64_t rpb = small ? 4 : 1;
  const int64_t blocks = (outs + rpb - 1) / rpb;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
#define VX_LAUNCH_MEAN(DT)                                                                      \
  do {                                                                                          \
    using T = Elem<DT>::T;                                                                      \
    if (small)                                                                                  \
      mean_dim_kernel<DT, 64><<<dim3((unsigned)blocks), 256, 0, stream>>>(                      \
          (const T*)in, (T*)out, s0, s1, s2, o0, o1, M, N, K);                                  \
    else                                                                                        \
      mean_dim_kernel<DT, 256><<<dim3((unsigned)blocks), 256, 0, stream>>>(                     \
          (const T*)in, (T*)out, s0, s1, s2, o0, o1, M, N, K);                                  \
  } while (0)
  switch (dtype) {
    case DT_F32: VX_LAUNCH_MEAN(DT_F32); break;
    case DT_BF16: VX_LAUNCH_MEAN(DT_BF16); break;
    case DT_F16: VX_LAUNCH_MEAN(DT_F16); break;
    default: return VX_ERR_UNSUPPORTED;
  }
#undef VX_LAUNCH_MEAN
  return launch_status();
}

int vx_rms_norm(const void* x, const void* residual, const void* weight, void* y, void* sum_out,
                int dtype, int64_t rows, int64_t n, int64_t x_stride, int64_t res_stride,
                int64_t y_stride, int64_t sum_stride, float eps, int mode, hipStream_t stream) {
  if (!x || !weight || !y || rows < 0 || n <= 0 || n > 0x7fffffff) return VX_ERR_ARG;
  if (mode != 0 && mode != 1) return VX_ERR_ARG;
  if (rows == 0) return VX_OK;
  const bool small = n <= 512;
  const int64_t rpb = small ? 4 : 1;
  const int64_t blocks = (rows + rpb - 1) / rpb;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
  if (dtype == DT_BF16 && n % 4 == 0 && n <= 8192 && ((x_stride | res_stride | y_stride | sum_stride) % 4 == 0) &&
      (((uintptr_t)x | (uintptr_t)residual | (uintptr_t)weight | (uintptr_t)y | (uintptr_t)sum_out) % 8 == 0)) {
#define VX_RMSV(GG, MV)                                                                            \
  rms_norm_bf16v_kernel<GG, MV><<<dim3((unsigned)blocks), 256, 0, stream>>>(                       \
      (const bf16_t*)x, (const bf16_t*)residual, (const bf16_t*)weight, (bf16_t*)y, (bf16_t*)sum_out, \
      rows, (int)n, x_stride, res_stride, y_stride, sum_stride, eps, mode)
    if (small) VX_RMSV(64, 2);
    else if (n <= 1024) VX_RMSV(256, 1);
    else if (n <= 2048) VX_RMSV(256, 2);
    else if (n <= 4096) VX_RMSV(256, 4);
    else VX_RMSV(256, 8);
#undef VX_RMSV
    return launch_status();
  }
#define VX_LAUNCH_RMS(DT)                                                                       \
  do {                                                                                          \
    using T = Elem<DT>::T;                                                                      \
    if (small)                                                                                  \
      rms_norm_kernel<DT, 64><<<dim3((unsigned)blocks), 256, 0, stream>>>(                      \
          (const T*)x, (const T*)residual, (const T*)weight, (T*)y, (T*)sum_out, rows, (int)n,  \
          x_stride, res_stride, y_stride, sum_stride, eps, mode);                               \
    else                                                                                        \
      rms_norm_kernel<DT, 256><<<dim3((unsigned)blocks), 256, 0, stream>>>(                     \
          (const T*)x, (const T*)residual, (const T*)weight, (T*)y, (T*)sum_out, rows, (int)n,  \
          x_stride, res_stride, y_stride, sum_stride, eps, mode);                               \
  } while (0)
  switch (dtype) {
    case DT_F32: VX_LAUNCH_RMS(DT_F32); break;
    case DT_BF16: VX_LAUNCH_RMS(DT_BF16); break;
    case DT_F16: VX_LAUNCH_RMS(DT_F16); break;
    default: return VX_ERR_UNSUPPORTED;
  }
#undef VX_LAUNCH_RMS
  return launch_status();
}

int64_t vx_log_softmax_workspace_bytes(int64_t rows, int64_t n) {
  if (rows < 0 || n <= 0) return 0;
  const int64_t nchunk = (n + LS_CHUNK - 1) / LS_CHUNK;
  return rows * nchunk * (int64_t)sizeof(LsPartial);
}

static int ls_partials(const void* x, int dtype, int64_t rows, int64_t n, int64_t xs, void* ws,
                       int64_t ws_bytes, hipStream_t stream, int* nchunk_out) {
  if (!x || !ws || rows < 0 || n <= 0 || n > 0x7fffffff - LS_CHUNK) return VX_ERR_ARG;
  if (rows > 65535) return VX_ERR_UNSUPPORTED;  // grid.y limit; callers split larger batches
  const int nchunk = (int)((n + LS_CHUNK - 1) / LS_CHUNK);
  if (ws_bytes < rows * nchunk * (int64_t)sizeof(LsPartial)) return VX_ERR_WORKSPACE;
  *nchunk_out = nchunk;
  if (rows == 0) return VX_OK;
  dim3 grid(nchunk, (unsigned)rows);
  switch (dtype) {
    case DT_F32:
      ls_partial_kernel<DT_F32><<<grid, LS_THREADS, 0, stream>>>((const float*)x, (LsPartial*)ws,
                                                                 (int)n, xs, nchunk);
      break;
    case DT_BF16:
      ls_partial_kernel<DT_BF16><<<grid, LS_THREADS, 0, stream>>>((const bf16_t*)x, (LsPartial*)ws,
                                                                  (int)n, xs, nchunk);
      break;
    case DT_F16:
      ls_partial_kernel<DT_F16><<<grid, LS_THREADS, 0, stream>>>((const _Float16*)x,
                                                                 (LsPartial*)ws, (int)n, xs, nchunk);
      break;
    default: return VX_ERR_UNSUPPORTED;
  }
  return launch_status();
}

int vx_log_softmax(const void* x, void* y, int dtype, int64_t rows, int64_t n, int64_t x_stride,
                   int64_t y_stride, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  if (!y) return VX_ERR_ARG;
  int nchunk = 0;
  int rc = ls_partials(x, dtype, rows, n, x_stride, workspace, workspace_bytes, stream, &nchunk);
  if (rc != VX_OK || rows == 0) return rc;
  const LsPartial* part = (const LsPartial*)workspace;
  const bool many = (int64_t)nchunk * rows >= 2048;  // thousands of (row, chunk) pairs: four chunks per workgroup
#define VX_LS_FINAL(DT, T)                                                                                         \
  do {                                                                                                             \
    if (many)                                                                                                      \
      ls_final_kernel<DT, 4><<<dim3((unsigned)((nchunk + 3) / 4), (unsigned)rows), LS_THREADS, 0, stream>>>(       \
          (const T*)x, (T*)y, part, (int)n, x_stride, y_stride, nchunk);                                           \
    else                                                                                                           \
      ls_final_kernel<DT, 1><<<dim3((unsigned)nchunk, (unsigned)rows), LS_THREADS, 0, stream>>>(                   \
          (const T*)x, (T*)y, part, (int)n, x_stride, y_stride, nchunk);                                           \
  } while (0)
  switch (dtype) {
    case DT_F32: VX_LS_FINAL(DT_F32, float); break;
    case DT_BF16: VX_LS_FINAL(DT_BF16, bf16_t); break;
    case DT_F16: VX_LS_FINAL(DT_F16, _Float16); break;
    default: return VX_ERR_UNSUPPORTED;
  }
#undef VX_LS_FINAL
  return launch_status();
}

int vx_logprobs(const void* logits, const int64_t* labels, float* out, int64_t* tokens_out,
                int dtype, int64_t rows, int64_t n, int64_t x_stride, void* workspace,
                int64_t workspace_bytes, hipStream_t stream) {
  if (!out) return VX_ERR_ARG;
  int nchunk = 0;
  int rc = ls_partials(logits, dtype, rows, n, x_stride, workspace, workspace_bytes, stream, &nchunk);
  if (rc != VX_OK || rows == 0) return rc;
  const unsigned blocks = (unsigned)rows;  // one wavefront per row
  const LsPartial* part = (const LsPartial*)workspace;
  switch (dtype) {
    case DT_F32:
      logprob_final_kernel<DT_F32><<<blocks, 64, 0, stream>>>((const float*)logits, labels, part, out,
                                                              tokens_out, rows, (int)n, x_stride,
                                                              nchunk);
      break;
    case DT_BF16:
      logprob_final_kernel<DT_BF16><<<blocks, 64, 0, stream>>>((const bf16_t*)logits, labels, part,
                                                               out, tokens_out, rows, (int)n,
                                                               x_stride, nchunk);
      break;
    case DT_F16:
      logprob_final_kernel<DT_F16><<<blocks, 64, 0, stream>>>((const _Float16*)logits, labels, part,
                                                              out, tokens_out, rows, (int)n,
                                                              x_stride, nchunk);
      break;
    default: return VX_ERR_UNSUPPORTED;
  }
  return launch_status();
}

static inline int64_t rms_bwd_blocks(int64_t rows, int64_t n) {
  const int64_t slots = n <= 128 ? 16 : 4;
  return std::max<int64_t>(1, std::min<int64_t>((rows + slots - 1) / slots, 512));
}
int64_t vx_rms_norm_bwd_workspace_bytes(int64_t rows, int64_t n) {
  if (rows < 0 || n <= 0) return 0;
  return rms_bwd_blocks(rows, n) * n * 4;
}
int vx_rms_norm_bwd(const void* x, const void* weight, const void* dy, void* dx, void* dw, int dtype, int64_t rows,
                    int64_t n, int64_t x_stride, int64_t dy_stride, int64_t dx_stride, float eps, int mode,
                    void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  if (!x || !weight || !dy || !dx || !dw || rows < 0 || n <= 0) return VX_ERR_ARG;
  if (mode != 0 && mode != 1) return VX_ERR_ARG;
  if ((dtype != DT_BF16 && dtype != DT_F16) || n % 8 != 0 || n > 8192 || (x_stride | dy_stride | dx_stride) % 8 != 0 ||
      (((uintptr_t)x | (uintptr_t)weight | (uintptr_t)dy | (uintptr_t)dx) % 16 != 0))
    return VX_ERR_UNSUPPORTED;
  const int64_t blocks = rms_bwd_blocks(rows, n);
  if (!workspace || workspace_bytes < blocks * n * 4) return VX_ERR_WORKSPACE;
  const size_t lds = (size_t)n * 4;
#define VX_RB(DT, G, MV)                                                                                            \
  rms_norm_bwd_kernel<DT, G, MV><<<(unsigned)blocks, 256, lds, stream>>>(                                          \
      (const Elem<DT>::T*)x, (const Elem<DT>::T*)weight, (const Elem<DT>::T*)dy, (Elem<DT>::T*)dx, (float*)workspace, \
      rows, (int)n, x_stride, dy_stride, dx_stride, eps, mode)
#define VX_RB_ANY(DT)                      \
  do {                                     \
    if (n <= 128) VX_RB(DT, 16, 1);        \
    else if (n <= 2048) VX_RB(DT, 64, 4);  \
    else VX_RB(DT, 64, 16);                \
  } while (0)
  if (rows > 0) {
    if (dtype == DT_BF16) VX_RB_ANY(DT_BF16); else VX_RB_ANY(DT_F16);
  }
#undef VX_RB_ANY
#undef VX_RB
  // no rows: the weight gradient is zero (no partial rows are read)
  const int nb = rows > 0 ? (int)blocks : 0;
  if (dtype == DT_BF16)
    rms_norm_bwd_finish_kernel<DT_BF16><<<(unsigned)((n + 63) / 64), 512, 0, stream>>>((const float*)workspace, nb, (int)n, (bf16_t*)dw);
  else
    rms_norm_bwd_finish_kernel<DT_F16><<<(unsigned)((n + 63) / 64), 512, 0, stream>>>((const float*)workspace, nb, (int)n, (_Float16*)dw);
  return launch_status();
}

int vx_logprobs_bwd(const void* logits, const int64_t* labels, const float* out, const float* d_out, void* d_logits,
                    int dtype, int64_t rows, int64_t n, int64_t x_stride, int64_t d_stride, hipStream_t stream) {
  if (!logits || !labels || !out || !d_out || !d_logits) return VX_ERR_ARG;
  if (rows < 0 || n <= 0 || n > 0x7fffffff) return VX_ERR_ARG;
  if (rows == 0) return VX_OK;
  if (rows > 65535) return VX_ERR_UNSUPPORTED;
  // Every workgroup must read the label's logit before any workgroup of the row overwrites it when the gradient goes
  // into the logits' memory: one workgroup per row then; else enough workgroups per row to fill the chip
  // "In place" is any overlap of the two ranges with equal pointers and strides; every other overlap is rejected
  // (a row's workgroups would read logits that another row's have already overwritten).
  const bool inplace = d_logits == logits;
  {
    const int64_t es = dtype == DT_F32 ? 4 : 2;
    const uintptr_t x0 = (uintptr_t)logits, x1 = x0 + (uintptr_t)(((rows - 1) * x_stride + n) * es);
    const uintptr_t d0 = (uintptr_t)d_logits, d1 = d0 + (uintptr_t)(((rows - 1) * d_stride + n) * es);
    const bool overlap = x0 < d1 && d0 < x1;
    if (overlap && !(inplace && x_stride == d_stride)) return VX_ERR_ARG;
  }
  const unsigned gx = inplace ? 1u : (unsigned)std::max<int64_t>(1, std::min<int64_t>((n + 2047) / 2048, 2048 / rows + 1));
  const dim3 grid(gx, (unsigned)rows);
  switch (dtype) {
    case DT_F32:
      logprob_bwd_kernel<DT_F32><<<grid, 256, 0, stream>>>((const float*)logits, labels, out, d_out, (float*)d_logits, (int)n,
                                                           x_stride, d_stride);
      break;
    case DT_BF16:
      logprob_bwd_kernel<DT_BF16><<<grid, 256, 0, stream>>>((const bf16_t*)logits, labels, out, d_out, (bf16_t*)d_logits,
                                                            (int)n, x_stride, d_stride);
      break;
    case DT_F16:
      logprob_bwd_kernel<DT_F16><<<grid, 256, 0, stream>>>((const _Float16*)logits, labels, out, d_out,
                                                           (_Float16*)d_logits, (int)n, x_stride, d_stride);
      break;
    default: return VX_ERR_UNSUPPORTED;
  }
  return launch_status();
}

int vx_logprobs_static(const void* logits, const int64_t* labels, float* out, int64_t* tokens_out,
                       int dtype, int64_t rows, int64_t n, int64_t x_stride, hipStream_t stream) {
  if (rows < 0 || n <= 0) return VX_ERR_ARG;
  // the size limit is checked before anything touches the device
  if (vx_log_softmax_workspace_bytes(rows, n) > kStaticScratchBytes) return VX_ERR_WORKSPACE;
  void* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc != VX_OK) return rc;
  // every partial the final kernel reads is written by the partial kernel of this call first, so
  // nothing in the array has to start at zero
  return vx_logprobs(logits, labels, out, tokens_out, dtype, rows, n, x_stride, ws, kStaticScratchBytes, stream);
}

}  // extern "C"
