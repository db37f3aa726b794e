// Token sampler: temperature, top-k, top-p and a seeded exponential race, one workgroup per row.
// Replaces Sampler.batch_sample_token (vexact/inferencer/sampler.py:29-113): the sort-based
// apply_top_k_top_p (:147-189) becomes two radix selects over the row (no sort, no softmax tensor,
// no probs / noise tensors), and the race argmax(probs / Exp(1)) (:115-145) is fused into the
// last pass.
//
// Everything a row's token depends on is a function of (that row's logits, temperature, k, p, seed,
// position): the noise is Philox4x32-10 keyed by the seed, with the position and the token index as
// the counter, so the token does not depend on the batch the row is in or on its place in it.
//
// The arithmetic is specified so that a CPU restatement can reproduce it bit for bit:
//   x_i   = f32(logit_i) * (1.0f / temperature)              (skipped for 1.0; a GPU tensor's div_ by a
//                                                          Python scalar multiplies by the fp32 reciprocal)
//   key_i = order-preserving uint32 image of x_i
//   top-k: T_k = k-th largest key; tokens with key < T_k are masked (ties at T_k all stay)
//   d_i   = x_i - max_j x_j ;  e_i = exp32(d_i) for d_i >= -32, else 0
//   w_i   = floor(e_i * 2^32) as an integer mass (0 for masked tokens)
//   top-p: Q = sum w_i, L = floor(f64(1.0f - p) * f64(Q)); T_p = smallest key whose inclusive
//          ascending mass sum_{key_j <= key} w_j exceeds L; tokens with key < T_p are masked. Equal
//          logits are kept or masked together (a sort keeps an arbitrary subset of a tie).
//   race:  token = argmin_i  E_i * exp32(-d_i)  over unmasked tokens with d_i >= -32, lowest index
//          on ties, E_i = -log32(u_i), u_i = (2 n_i + 1) / 2^33, n_i = Philox output for token i
// exp32 / log32 are fixed polynomial evaluations in fp32 made of IEEE add / mul / div only (this file
// is compiled without contraction), integer sums are order-free, so any tiling gives the same bits.
#include <type_traits>

#include "common.h"

namespace vx {

constexpr int SM_THREADS = 1024;
constexpr int SM_WAVES = SM_THREADS / 64;
constexpr float SM_CUTOFF = -32.0f;
// Radix digits of the 32-bit keys, most significant first: 12 + 10 + 10 bits. The wide first digit
// (sign, exponent, three mantissa bits) spreads a row of logits over a few hundred bins, which keeps
// the LDS atomics of the first pass from piling onto a handful of addresses.
constexpr int SM_BINS0 = 4096;

__device__ __forceinline__ uint32_t float_key(float x) {
  const uint32_t b = __builtin_bit_cast(uint32_t, x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// exp(d) for |d| <= 32: n = rint(d * log2 e), r = (d - n ln2_hi) - n ln2_lo, degree-7 Taylor, * 2^n
__device__ __forceinline__ float exp32(float d) {
  const float n = rintf(d * 1.44269502162933349609375f);
  const float r = (d - n * 0.693145751953125f) - n * 1.428606765330187045037746429443359375e-06f;
  float p = 1.0f / 5040.0f;
  p = p * r + 1.0f / 720.0f;
  p = p * r + 1.0f / 120.0f;
  p = p * r + 1.0f / 24.0f;
  p = p * r + 1.0f / 6.0f;
  p = p * r + 0.5f;
  p = p * r + 1.0f;
  p = p * r + 1.0f;
  return __builtin_bit_cast(float, __builtin_bit_cast(int32_t, p) + (int32_t)n * (1 << 23));
}

// -log((2 n + 1) / 2^33): f = f32(2 n + 1) = 2^e * m, m in [sqrt(1/2), sqrt 2), s = (m-1)/(m+1),
// log m = 2 s (1 + s^2/3 + s^4/5 + s^6/7 + s^8/9)
__device__ __forceinline__ float neg_log_uniform(uint32_t n) {
  const float f = (float)(2ull * (uint64_t)n + 1ull);
  const uint32_t b = __builtin_bit_cast(uint32_t, f);
  int e = (int)(b >> 23) - 127;
  float m = __builtin_bit_cast(float, (b & 0x007fffffu) | 0x3f800000u);
  if (m > 1.41421353816986083984375f) {
    m = m * 0.5f;
    e += 1;
  }
  const float s = (m - 1.0f) / (m + 1.0f);
  const float s2 = s * s;
  float q = 1.0f / 9.0f;
  q = q * s2 + 1.0f / 7.0f;
  q = q * s2 + 1.0f / 5.0f;
  q = q * s2 + 1.0f / 3.0f;
  q = q * s2 + 1.0f;
  const float logm = (2.0f * s) * q;
  return (float)(33 - e) * 0.693147182464599609375f - logm;
}

// Philox4x32-10 (Salmon et al., SC'11)
__device__ __forceinline__ uint4 philox4x32(uint4 c, uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; r++) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c.x;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c.z;
    c = make_uint4((uint32_t)(p1 >> 32) ^ c.y ^ k0, (uint32_t)p1, (uint32_t)(p0 >> 32) ^ c.w ^ k1, (uint32_t)p0);
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c;
}

struct SampleParams {
  const void* logits;
  int dtype;  // 0 bf16, 1 fp32
  int64_t ld;
  int V;
  float temperature;
  int top_k;    // <= 0 or >= V: off
  float top_p;  // >= 1: off
  const int64_t* seeds;
  const int64_t* positions;
  int64_t* tokens;
};

// four consecutive tokens 4 g .. 4 g + 3 of the row, as x = logit * (1 / temperature); tokens past V get ok = false
struct Quad {
  float x[4];
  bool ok[4];
};
__device__ __forceinline__ Quad load_quad(const SampleParams& p, const void* row, bool aligned, int g) {
  Quad q;
  const int i0 = 4 * g;
  if (p.dtype == 0) {
    const bf16_t* r = (const bf16_t*)row + i0;
    if (aligned && i0 + 3 < p.V) {
      const uint2 v = *(const uint2*)r;
      q.x[0] = bf16lo(v.x); q.x[1] = bf16hi(v.x); q.x[2] = bf16lo(v.y); q.x[3] = bf16hi(v.y);
      q.ok[0] = q.ok[1] = q.ok[2] = q.ok[3] = true;
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        q.ok[j] = i0 + j < p.V;
        q.x[j] = q.ok[j] ? bf16_to_f32(r[j]) : 0.f;
      }
    }
  } else {
    const float* r = (const float*)row + i0;
    if (aligned && i0 + 3 < p.V) {
      const float4 v = *(const float4*)r;
      q.x[0] = v.x; q.x[1] = v.y; q.x[2] = v.z; q.x[3] = v.w;
      q.ok[0] = q.ok[1] = q.ok[2] = q.ok[3] = true;
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        q.ok[j] = i0 + j < p.V;
        q.x[j] = q.ok[j] ? r[j] : 0.f;
      }
    }
  }
  if (p.temperature != 1.0f) {
    const float inv = 1.0f / p.temperature;
#pragma unroll
    for (int j = 0; j < 4; j++) q.x[j] = q.x[j] * inv;
  }
  return q;
}

// Calls f(quad, group, in_range) for every group of the row, SM_UNROLL groups per thread and trip,
// all of a trip's loads issued before the first is used. Every thread makes the same number of
// calls (in_range = false past the end), so f may vote across the wavefront.
constexpr int SM_UNROLL = 4;
template <class Fn>
__device__ __forceinline__ void scan_row(const SampleParams& p, const void* row, bool aligned, int groups, Fn f) {
  for (int g0 = 0; g0 < groups; g0 += SM_THREADS * SM_UNROLL) {
    Quad q[SM_UNROLL];
#pragma unroll
    for (int u = 0; u < SM_UNROLL; u++) {
      const int g = g0 + u * SM_THREADS + (int)threadIdx.x;
      q[u] = load_quad(p, row, aligned, g < groups ? g : 0);
    }
#pragma unroll
    for (int u = 0; u < SM_UNROLL; u++) {
      const int g = g0 + u * SM_THREADS + (int)threadIdx.x;
      f(q[u], g, g < groups);
    }
  }
}

__device__ __forceinline__ uint64_t wave_sum_u64(uint64_t v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint32_t lo = __shfl_xor((uint32_t)v, o, 64), hi = __shfl_xor((uint32_t)(v >> 32), o, 64);
    v += ((uint64_t)hi << 32) | lo;
  }
  return v;
}

// hist[bin] += w for the lanes with valid set. When every valid lane of the wavefront hits one bin
// (the common case for the leading digits of float keys) the wavefront adds once.
template <bool COUNT>  // COUNT: every w is 1
__device__ __forceinline__ void hist_add(unsigned long long* hist, bool valid, uint32_t bin, uint64_t w) {
  const uint64_t mask = __ballot(valid);
  if (mask == 0) return;
  const int leader = __ffsll((long long)mask) - 1;
  const uint32_t b0 = __shfl(bin, leader, 64);
  if (__ballot(valid && bin != b0) == 0) {
    const uint64_t s = COUNT ? (uint64_t)__popcll(mask) : wave_sum_u64(valid ? w : 0ull);
    if ((int)(threadIdx.x & 63) == leader) atomicAdd(&hist[b0], (unsigned long long)s);
  } else if (valid) {
    atomicAdd(&hist[bin], (unsigned long long)w);
  }
}

// Wavefront 0: first bin b (0..nbins-1) whose inclusive prefix sum reaches target; writes b and the
// exclusive prefix at b to res[0], res[1]. If the total is below target, the last non-empty bin.
// Lane l owns the nbins / 64 consecutive bins starting at l * nbins / 64.
__device__ __forceinline__ void pick_bin(const unsigned long long* hist, int nbins, uint64_t target,
                                         unsigned long long* res) {
  const int lane = threadIdx.x & 63;
  const int per = nbins >> 6;
  const unsigned long long* mine = hist + lane * per;
  uint64_t local = 0;
  for (int j = 0; j < per; j++) local += mine[j];
  uint64_t incl = local;  // inclusive scan over lanes
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const uint32_t lo = __shfl_up((uint32_t)incl, o, 64), hi = __shfl_up((uint32_t)(incl >> 32), o, 64);
    if (lane >= o) incl += ((uint64_t)hi << 32) | lo;
  }
  const uint64_t hit = __ballot(incl >= target);
  const uint64_t nonempty = __ballot(local != 0);
  const bool fallback = hit == 0;
  const int pick_lane = !fallback ? __ffsll((long long)hit) - 1 : (nonempty ? 63 - __builtin_clzll(nonempty) : 0);
  if (lane == pick_lane) {
    uint64_t ex = incl - local;
    int j = 0;
    if (!fallback) {
      while (j < per - 1 && ex + mine[j] < target) ex += mine[j++];
    } else {
      int last = per - 1;
      while (last > 0 && mine[last] == 0) last--;
      while (j < last) ex += mine[j++];
    }
    res[0] = (unsigned long long)(lane * per + j);
    res[1] = (unsigned long long)ex;
  }
}

__global__ __launch_bounds__(SM_THREADS) void sample_kernel(SampleParams p) {
  __shared__ unsigned long long hist[SM_BINS0];
  __shared__ unsigned long long res[2];
  __shared__ float redf[SM_WAVES];
  __shared__ unsigned long long red64[SM_WAVES];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t rowi = blockIdx.x;
  const void* row = (const char*)p.logits + rowi * p.ld * (p.dtype == 0 ? 2 : 4);
  const bool aligned = ((uintptr_t)row & (p.dtype == 0 ? 7 : 15)) == 0;
  const int groups = (p.V + 3) >> 2;

  // ---- row maximum of x
  float mx = -INFINITY;
  scan_row(p, row, aligned, groups, [&](const Quad& q, int, bool in) {
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (in && q.ok[j]) mx = fmaxf(mx, q.x[j]);
  });
  mx = block_max<SM_WAVES>(mx, redf);

  // ---- radix selects, most significant digit first. desc: by count from the top (top-k);
  // otherwise by mass from the bottom over keys >= floor_key (top-p).
  auto radix_select = [&](auto desc_tag, uint64_t target, uint32_t floor_key) -> uint32_t {
    constexpr bool desc = decltype(desc_tag)::value;
    uint32_t prefix = 0;
    for (int pass = 0; pass < 3; pass++) {
      const int shift = pass == 0 ? 20 : (pass == 1 ? 10 : 0);
      const int bits = pass == 0 ? 12 : 10;
      const int nbins = 1 << bits;
      for (int i = tid; i < nbins; i += SM_THREADS) hist[i] = 0;
      __syncthreads();
      scan_row(p, row, aligned, groups, [&](const Quad& q, int, bool in) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          bool valid = in && q.ok[j];
          uint32_t key = 0;
          uint64_t w = 1;
          if (valid) {
            key = float_key(q.x[j]);
            if (pass > 0 && (key >> (shift + bits)) != prefix) valid = false;
            if constexpr (!desc) {
              const float d = q.x[j] - mx;
              if (key < floor_key || !(d >= SM_CUTOFF)) valid = false;
              else w = (uint64_t)(exp32(d) * 4294967296.0f);
            }
          }
          uint32_t bin = (key >> shift) & (uint32_t)(nbins - 1);
          if (desc) bin = (uint32_t)(nbins - 1) - bin;
          hist_add<desc>(hist, valid, bin, w);
        }
      });
      __syncthreads();
      if (!desc && pass == 0) {  // the mass limit needs the total first: L = floor((1 - p) Q), target = L + 1
        if (wave == 0) {
          uint64_t s = 0;
          for (int j = 0; j < nbins / 64; j++) s += hist[lane * (nbins / 64) + j];
          s = wave_sum_u64(s);
          if (lane == 0) red64[0] = s;
        }
        __syncthreads();
        const double lim = (double)(1.0f - p.top_p) * (double)red64[0];
        target = (uint64_t)lim + 1ull;
      }
      if (wave == 0) pick_bin(hist, nbins, target, res);
      __syncthreads();
      uint32_t b = (uint32_t)res[0];
      target -= res[1];
      if (desc) b = (uint32_t)(nbins - 1) - b;
      prefix = (prefix << bits) | b;
      __syncthreads();
    }
    return prefix;
  };

  uint32_t thr = 0;
  if (p.top_k > 0 && p.top_k < p.V) thr = radix_select(std::true_type{}, (uint64_t)p.top_k, 0u);
  if (p.top_p < 1.0f) {
    const uint32_t tp = radix_select(std::false_type{}, 0ull, thr);
    thr = tp > thr ? tp : thr;
  }

  // ---- the race over the surviving tokens
  const uint64_t seed = (uint64_t)p.seeds[rowi], pos = (uint64_t)p.positions[rowi];
  float best = INFINITY;
  int best_i = 0x7fffffff;
  scan_row(p, row, aligned, groups, [&](const Quad& q, int g, bool in) {
    bool any = false;
    bool live[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      live[j] = in && q.ok[j] && float_key(q.x[j]) >= thr && (q.x[j] - mx) >= SM_CUTOFF;
      any |= live[j];
    }
    if (!any) return;
    const uint4 r = philox4x32(make_uint4((uint32_t)g, (uint32_t)pos, (uint32_t)(pos >> 32), 0u), (uint32_t)seed,
                               (uint32_t)(seed >> 32));
    const uint32_t rn[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      if (!live[j]) continue;
      const float s = neg_log_uniform(rn[j]) * exp32(mx - q.x[j]);
      if (s < best) {  // a thread visits its tokens in ascending order, so strict < keeps the lowest index
        best = s;
        best_i = 4 * g + j;
      }
    }
  });
  // (score, index) minimum: non-negative floats order like their bit patterns
  unsigned long long packed = ((unsigned long long)__builtin_bit_cast(uint32_t, best) << 32) | (uint32_t)best_i;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint32_t lo = __shfl_xor((uint32_t)packed, o, 64), hi = __shfl_xor((uint32_t)(packed >> 32), o, 64);
    const unsigned long long other = ((unsigned long long)hi << 32) | lo;
    packed = other < packed ? other : packed;
  }
  if (lane == 0) red64[wave] = packed;
  __syncthreads();
  if (tid == 0) {
    unsigned long long m = red64[0];
    for (int w = 1; w < SM_WAVES; w++) m = red64[w] < m ? red64[w] : m;
    const uint32_t tok = (uint32_t)m;
    p.tokens[rowi] = tok < (uint32_t)p.V ? (int64_t)tok : 0;  // a row of NaN / -inf has no live token
  }
}

}  // namespace vx

extern "C" int vx_sample_tokens(const void* logits, int dtype, int64_t ld, int64_t rows, int64_t V, float temperature,
                                int top_k, float top_p, const int64_t* seeds, const int64_t* positions,
                                int64_t* tokens_out, hipStream_t stream) {
  using namespace vx;
  if (rows == 0) return VX_OK;
  if (!logits || !seeds || !positions || !tokens_out || rows < 0 || V <= 0 || V > 0x7ffffff0LL || ld < V) return VX_ERR_ARG;
  if (dtype != 0 && dtype != 1) return VX_ERR_UNSUPPORTED;
  if (!(temperature > 0.f) || !(top_p > 0.f)) return VX_ERR_ARG;  // greedy decoding is vx_logprobs' argmax
  if (rows > 0x7fffffffLL) return VX_ERR_ARG;
  SampleParams p{logits, dtype, ld, (int)V, temperature, top_k, top_p, seeds, positions, tokens_out};
  sample_kernel<<<dim3((unsigned)rows), SM_THREADS, 0, stream>>>(p);
  return launch_status();
}
