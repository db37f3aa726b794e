// bf16 "NT" GEMM building blocks shared by the dense GEMM and the MoE grouped GEMMs:
//   C[m, n] = r16( sum_k X[m, k] * W[n, k]  (+ bias[n]) ),  X and W both K-contiguous.
//
// Two kernels, identical arithmetic per output element:
//   * gemm_stream_kernel  - few rows (<= 64 per tile): every wavefront streams its own 16
//     weight rows straight from HBM into registers; only the activation tile goes through LDS.
//   * gemm_tiled_kernel   - many rows: classic 128x128x64 LDS-tiled, double buffered.
// In both, the MFMA A operand is a 16x32 weight fragment, the B operand a 32x16 activation
// fragment, and each accumulator walks K in ascending 32-wide chunks (zero padded past K), so
// a row's result does not depend on which kernel, tile size or neighbour rows it ran with.
//
// Grouped mode (MoE): row tiles come from a tile table (expert id, first row, row count) built
// on the device by the routing kernel, activation rows may be gathered through row_src, and
// the SWIGLU epilogue fuses gate/up projections:  out = r16(r16(r16(silu(r16(g))) * r16(u)) * w_row).
#pragma once
#include "common.h"

namespace vx {

enum : int { EPI_PLAIN = 0, EPI_SWIGLU = 1 };

struct GemmParams {
  const bf16_t* x;   // activations
  int64_t ldx;
  const bf16_t* w;   // weights [N, K] (EPI_SWIGLU: gate rows)
  const bf16_t* w2;  // EPI_SWIGLU: up rows
  int64_t ldw;
  int64_t w_gstride;  // elements between consecutive groups' weights
  const bf16_t* bias;  // [N] or null (EPI_PLAIN only)
  bf16_t* c;
  int64_t ldc;
  int M, N, K;
  // grouped mode
  const int* tile_group;  // [m_tiles] group id, -1 = unused tile
  const int* tile_row0;   // [m_tiles] first row of the tile (in C / sorted order)
  const int* tile_rows;   // [m_tiles] rows in the tile
  const int* row_src;     // [M] row of x feeding C row i (null = identity)
  const bf16_t* row_scale;      // EPI_SWIGLU: per-row routing weight (null = none), looked up as
  const int* row_scale_idx;     //   row_scale[row_scale_idx[i]] (idx null = identity)
};

__device__ __forceinline__ float silu_f32(float g) { return g / (1.0f + expf(-g)); }

// out = r16(r16(r16(silu(r16(g))) * r16(u)) * w)
__device__ __forceinline__ bf16_t swiglu_bf16(float g, float u, float w) {
  const float gb = bf16_to_f32(f32_to_bf16(g));
  const float ub = bf16_to_f32(f32_to_bf16(u));
  const float a = bf16_to_f32(f32_to_bf16(silu_f32(gb)));
  const float h = bf16_to_f32(f32_to_bf16(a * ub));
  return f32_to_bf16(h * w);
}

// ---------------------------------------------------------------------------------------
// Streaming kernel. 64 NW threads = NW wavefronts (4 unless said otherwise); wavefront v owns weight rows
// [n0 + 16 v, n0 + 16 v + 16); the block covers 16 NW weight rows and BM = 16*MT activation rows.
// NW = 1 is for launches of a few tiles (a single token's eight experts): four times the workgroups, so that
// the weight stream is pulled by every CU instead of the hundred that 4-wavefront blocks would occupy.
// ---------------------------------------------------------------------------------------
// U  = k-steps of weight loads a wavefront keeps in flight (one group);
// KD = divisor of the staged K chunk: KC = 32768 / (BM * KD) elements per LDS fill (64 KB / KD of
//      LDS per block, so KD = 2 lets more blocks share a CU). 32 U must divide KC.
// PACKED: the weights are in fragment order (pack_weights_kernel): the 1 KB that the 64 lanes of a
// wavefront feed to one MFMA (16 weight rows x 32 k) is contiguous and in lane order, so a wavefront
// streams one linear run of (K / 32) KB per 16-row block instead of 16 rows of pitch ldw. p.ldw is then
// the number of 32-wide k-chunks stored per row block (K rounded up to a multiple of 32 U, zero filled).
template <int MT, int EPI, bool GROUPED, int U = 8, int KD = 1, bool PACKED = false, int NW = 4>
__global__ __launch_bounds__(64 * NW) void gemm_stream_kernel(GemmParams p) {
  constexpr int NT = 64 * NW;  // threads
  constexpr int BM = 16 * MT;
  constexpr int KC = 32768 / (BM * KD);  // K elements staged per LDS fill
  constexpr int RB = KC * 2 + 16;        // +16: rows land on distinct bank groups
  __shared__ __attribute__((aligned(16))) uint8_t xs[BM * RB];
  static_assert(KC % (32 * U) == 0, "a staged chunk must hold whole groups");
  static_assert(!PACKED || 8 % U == 0, "a fragment-order image is zero-filled to multiples of 8 k-chunks: a group of U chunks must not cross that");

  int row0, rows;
  int64_t wbase = 0;
  if constexpr (GROUPED) {
    const int t = blockIdx.y;
    const int grp = p.tile_group[t];
    if (grp < 0) return;
    row0 = p.tile_row0[t];
    rows = p.tile_rows[t];
    wbase = (int64_t)grp * p.w_gstride;
  } else {
    row0 = blockIdx.y * BM;
    rows = min(BM, p.M - row0);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (16 * NW) + wave * 16;
  const int K = p.K;
  const bf16_t* wp;
  const bf16_t* wp2 = nullptr;
  if constexpr (PACKED) {
    const int64_t woff = wbase + (int64_t)min(n0 >> 4, ((p.N + 15) >> 4) - 1) * p.ldw * 512 + lane * 8;
    wp = p.w + woff;
    if constexpr (EPI == EPI_SWIGLU) wp2 = p.w2 + woff;
  } else {
    const int nrow = min(n0 + r16, p.N - 1);
    wp = p.w + wbase + (int64_t)nrow * p.ldw + 8 * g;
    if constexpr (EPI == EPI_SWIGLU) wp2 = p.w2 + wbase + (int64_t)nrow * p.ldw + 8 * g;
  }

  f32x4 acc[MT], acc2[EPI == EPI_SWIGLU ? MT : 1];
#pragma unroll
  for (int i = 0; i < MT; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  if constexpr (EPI == EPI_SWIGLU) {
#pragma unroll
    for (int i = 0; i < MT; i++) acc2[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  uint4 wa[U], wb[EPI == EPI_SWIGLU ? U : 1];
  // Weight loads of one group of U k-steps. A group that lies fully inside K is loaded without any
  // masking so the loads stay in flight across the MFMAs of the previous group; only a ragged last
  // group (K not a multiple of 32*U) pays for masks, and a group past K is all zeros.
  auto load_w = [&](int kstep0) {
    if constexpr (PACKED) {  // chunk c of the row block lies at 512 c elements; stored chunks past K are zero
      if (kstep0 < K) {
#pragma unroll
        for (int u = 0; u < U; u++) {
          wa[u] = ldg16_raw(wp + (int64_t)(kstep0 + 32 * u) * 16);
          if constexpr (EPI == EPI_SWIGLU) wb[u] = ldg16_raw(wp2 + (int64_t)(kstep0 + 32 * u) * 16);
        }
      } else {
#pragma unroll
        for (int u = 0; u < U; u++) {
          wa[u] = make_uint4(0, 0, 0, 0);
          if constexpr (EPI == EPI_SWIGLU) wb[u] = make_uint4(0, 0, 0, 0);
        }
      }
    } else if (kstep0 + 32 * U <= K) {
#pragma unroll
      for (int u = 0; u < U; u++) {
        wa[u] = ldg16_raw(wp + kstep0 + 32 * u);
        if constexpr (EPI == EPI_SWIGLU) wb[u] = ldg16_raw(wp2 + kstep0 + 32 * u);
      }
    } else if (kstep0 < K) {
#pragma unroll
      for (int u = 0; u < U; u++) {
        const bool ok = kstep0 + 32 * u + 8 * g < K;
        // a piece past K is never dereferenced: the row's first piece is read instead (wp already points 8 g in)
        const int ko = ok ? kstep0 + 32 * u : -8 * g;
        wa[u] = ldg16(wp + ko, ok);
        if constexpr (EPI == EPI_SWIGLU) wb[u] = ldg16(wp2 + ko, ok);
      }
    } else {
#pragma unroll
      for (int u = 0; u < U; u++) {
        wa[u] = make_uint4(0, 0, 0, 0);
        if constexpr (EPI == EPI_SWIGLU) wb[u] = make_uint4(0, 0, 0, 0);
      }
    }
  };

  // Activation staging: thread owns pieces tid + NT j (j < NP) of the BM x KC tile; piece =
  // (row pc / PPR, 16-byte column pc % PPR). Row sources are resolved once.
  constexpr int PPR = KC / 8;            // 16-byte pieces per staged row
  constexpr int NP = BM * PPR / NT;      // pieces per thread
  static_assert(BM * PPR % NT == 0, "pieces must split evenly over the threads");
  int64_t xoff[NP];                      // element offset of the piece's row in x, -1 = zero row
#pragma unroll
  for (int j = 0; j < NP; j++) {
    const int pc = threadIdx.x + NT * j;
    const int r = pc / PPR;
    int64_t off = -1;
    if (r < rows) {
      const int64_t sr = p.row_src ? (int64_t)p.row_src[row0 + r] : (int64_t)(row0 + r);
      off = sr * p.ldx + (pc % PPR) * 8;
    }
    xoff[j] = off;
  }

  // The activation chunk for step c+1 is requested before the MFMAs of chunk c and written to LDS
  // after them, so its latency hides behind compute instead of stalling every wavefront at a barrier.
  uint4 stage[NP];
  auto stage_load = [&](int kc) {
#pragma unroll
    for (int j = 0; j < NP; j++) {  // all loads of the fill in flight together
      const int c8 = (threadIdx.x + NT * j) % PPR;
      const bool ok = xoff[j] >= 0 && kc + c8 * 8 < K;
      stage[j] = ldg16_raw(p.x + (ok ? xoff[j] + kc : 0));
    }
  };
  auto stage_store = [&](int kc) {
#pragma unroll
    for (int j = 0; j < NP; j++) {
      const int pc = threadIdx.x + NT * j;
      const int c8 = pc % PPR;
      const bool ok = xoff[j] >= 0 && kc + c8 * 8 < K;
      *(uint4*)(xs + (pc / PPR) * RB + c8 * 16) = mask16(stage[j], ok);
    }
  };

  load_w(0);
  stage_load(0);
  stage_store(0);
  __syncthreads();
  for (int kc = 0; kc < K; kc += KC) {
    const bool more = kc + KC < K;
    if (more) stage_load(kc + KC);
    const int kend = min(K - kc, KC);
    for (int s0 = 0; s0 < kend; s0 += 32 * U) {
      uint4 ca[U], cb[EPI == EPI_SWIGLU ? U : 1];
#pragma unroll
      for (int u = 0; u < U; u++) {
        ca[u] = wa[u];
        if constexpr (EPI == EPI_SWIGLU) cb[u] = wb[u];
      }
      load_w(kc + s0 + 32 * U);  // next group (zero past K); stays in flight during the MFMAs
#pragma unroll
      for (int u = 0; u < U; u++) {
#pragma unroll
        for (int i = 0; i < MT; i++) {
          const uint4 xf = *(const uint4*)(xs + (16 * i + r16) * RB + (s0 + 32 * u + 8 * g) * 2);
          acc[i] = mfma16(ca[u], xf, acc[i]);
          if constexpr (EPI == EPI_SWIGLU) acc2[i] = mfma16(cb[u], xf, acc2[i]);
        }
      }
    }
    if (more) {
      __syncthreads();  // everyone is done reading this chunk
      stage_store(kc + KC);
      __syncthreads();
    }
  }

  // lane holds C[row 16 i + r16][col n0 + 4 g + j], j = 0..3
  const int nc = n0 + 4 * g;
#pragma unroll
  for (int i = 0; i < MT; i++) {
    const int m = 16 * i + r16;
    if (m >= rows) continue;
    const int64_t orow = row0 + m;
    bf16_t o[4];
    if constexpr (EPI == EPI_SWIGLU) {
      float wr = 1.0f;  // no row scale: the last rounding of swiglu_bf16 is then the identity
      if (p.row_scale) wr = bf16_to_f32(p.row_scale[p.row_scale_idx ? p.row_scale_idx[orow] : (int)orow]);
#pragma unroll
      for (int j = 0; j < 4; j++) o[j] = swiglu_bf16(acc[i][j], acc2[i][j], wr);
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        float v = acc[i][j];
        if (p.bias && nc + j < p.N) v += bf16_to_f32(p.bias[nc + j]);
        o[j] = f32_to_bf16(v);
      }
    }
    bf16_t* cp = p.c + orow * p.ldc + nc;
    if (nc + 3 < p.N && ((p.ldc & 3) == 0)) {
      uint2 pk;
      pk.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
      pk.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
      *(uint2*)cp = pk;
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (nc + j < p.N) cp[j] = o[j];
    }
  }
}

// ---------------------------------------------------------------------------------------
// Tiled kernel: 128 activation rows x 128 weight rows x 64 K per step, 4 wavefronts in a
// 2 (rows) x 2 (cols) arrangement, each computing 64x64 as 4x4 MFMA tiles. Global loads for
// step t+1 are issued before the MFMAs of step t and written to the other LDS buffer after.
// EPI_SWIGLU: weight tile rows 0..63 are gate rows n0..n0+63 and rows 64..127 the matching up
// rows; wavefront column wn then owns gate rows [32 wn, +32) and the same up rows, so the
// block produces 64 output columns.
// ---------------------------------------------------------------------------------------
constexpr int TL_BM = 128, TL_BN = 128, TL_BK = 64;
constexpr int TL_RB = TL_BK * 2 + 16;  // 144-byte LDS rows

template <int EPI, bool GROUPED>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(GemmParams p) {
  __shared__ __attribute__((aligned(16))) uint8_t lx[2][TL_BM * TL_RB];
  __shared__ __attribute__((aligned(16))) uint8_t lw[2][TL_BN * TL_RB];

  int row0, rows;
  int64_t wbase = 0;
  if constexpr (GROUPED) {
    const int t = blockIdx.y;
    const int grp = p.tile_group[t];
    if (grp < 0) return;
    row0 = p.tile_row0[t];
    rows = p.tile_rows[t];
    wbase = (int64_t)grp * p.w_gstride;
  } else {
    row0 = blockIdx.y * TL_BM;
    rows = min(TL_BM, p.M - row0);
  }
  constexpr int NOUT = (EPI == EPI_SWIGLU) ? 64 : 128;  // output columns per block
  const int n0 = blockIdx.x * NOUT;
  const int K = p.K, N = p.N;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;

  // global -> LDS staging: thread handles pieces tid + 256 j, piece = (row = pc / 8, c8 = pc % 8)
  const bf16_t* xrow[4];
  const bf16_t* wrow[4];
  bool xok[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int pc = tid + 256 * j;
    const int r = pc >> 3, c8 = pc & 7;
    xok[j] = r < rows;
    int64_t src = 0;
    if (xok[j]) src = p.row_src ? (int64_t)p.row_src[row0 + r] : (int64_t)(row0 + r);
    xrow[j] = p.x + src * p.ldx + c8 * 8;
    int wr;
    const bf16_t* wb = p.w;
    if constexpr (EPI == EPI_SWIGLU) {
      wr = n0 + (r & 63);
      if (r >= 64) wb = p.w2;
    } else {
      wr = n0 + r;
    }
    wr = min(wr, N - 1);
    wrow[j] = wb + wbase + (int64_t)wr * p.ldw + c8 * 8;
  }
  uint4 gx[4], gw[4];
  auto gload = [&](int k0) {  // raw loads; zeroing happens in lstore, after the MFMAs of this step
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int c8 = (tid + 256 * j) & 7;
      // a piece past K is never dereferenced: the row's first piece is read instead (the row pointers already
      // point 8 c8 in), since with K < 64 even k0 = 0 would reach past the row, and past the tensor in its last rows
      const int ko = (k0 + c8 * 8 < K) ? k0 : -8 * c8;
      gx[j] = ldg16_raw(xrow[j] + ko);
      gw[j] = ldg16_raw(wrow[j] + ko);
    }
  };
  auto lstore = [&](int buf, int k0) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int pc = tid + 256 * j;
      const int r = pc >> 3, c8 = pc & 7;
      const bool kok = k0 + c8 * 8 < K;
      *(uint4*)(&lx[buf][r * TL_RB + c8 * 16]) = mask16(gx[j], xok[j] && kok);
      *(uint4*)(&lw[buf][r * TL_RB + c8 * 16]) = mask16(gw[j], kok);
    }
  };

  f32x4 acc[4][4];  // [m tile][n tile]
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // LDS row of weight n-tile j for this wavefront
  auto wtile_row = [&](int j) {
    if constexpr (EPI == EPI_SWIGLU) return (j < 2 ? 0 : 64) + 32 * wn + 16 * (j & 1);
    else return 64 * wn + 16 * j;
  };

  const int nk = (K + TL_BK - 1) / TL_BK;
  gload(0);
  lstore(0, 0);
  __syncthreads();
  for (int kt = 0; kt < nk; kt++) {
    const int buf = kt & 1;
    if (kt + 1 < nk) gload((kt + 1) * TL_BK);
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      uint4 wf[4], xf[4];
#pragma unroll
      for (int j = 0; j < 4; j++)
        wf[j] = *(const uint4*)(&lw[buf][(wtile_row(j) + r16) * TL_RB + (32 * ks + 8 * g) * 2]);
#pragma unroll
      for (int i = 0; i < 4; i++)
        xf[i] = *(const uint4*)(&lx[buf][(64 * wm + 16 * i + r16) * TL_RB + (32 * ks + 8 * g) * 2]);
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = mfma16(wf[j], xf[i], acc[i][j]);
    }
    if (kt + 1 < nk) lstore(buf ^ 1, (kt + 1) * TL_BK);
    __syncthreads();
  }

  // epilogue: lane holds C[row 64 wm + 16 i + r16][col (tile j) + 4 g + c]
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int m = 64 * wm + 16 * i + r16;
    if (m >= rows) continue;
    const int64_t orow = row0 + m;
    if constexpr (EPI == EPI_SWIGLU) {
      float wr = 1.0f;  // no row scale: the last rounding of swiglu_bf16 is then the identity
      if (p.row_scale) wr = bf16_to_f32(p.row_scale[p.row_scale_idx ? p.row_scale_idx[orow] : (int)orow]);
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int nc = n0 + 32 * wn + 16 * j + 4 * g;
        bf16_t* cp = p.c + orow * p.ldc + nc;
#pragma unroll
        for (int c = 0; c < 4; c++)
          if (nc + c < N) cp[c] = swiglu_bf16(acc[i][j][c], acc[i][j + 2][c], wr);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int nc = n0 + 64 * wn + 16 * j + 4 * g;
        bf16_t* cp = p.c + orow * p.ldc + nc;
        bf16_t o[4];
#pragma unroll
        for (int c = 0; c < 4; c++) {
          float v = acc[i][j][c];
          if (p.bias && nc + c < N) v += bf16_to_f32(p.bias[nc + c]);
          o[c] = f32_to_bf16(v);
        }
        if (nc + 3 < N && ((p.ldc & 3) == 0)) {
          uint2 pk;
          pk.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
          pk.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
          *(uint2*)cp = pk;
        } else {
#pragma unroll
          for (int c = 0; c < 4; c++)
            if (nc + c < N) cp[c] = o[c];
        }
      }
    }
  }
}

// Host-side checks shared by the dense and grouped entry points: 16-byte loads need K-contiguous
// operands whose rows start on 16-byte boundaries.
static inline bool gemm_fast_ok(const void* x, const void* w, int64_t K, int64_t ldx, int64_t ldw) {
  return (K % 8 == 0) && (ldx % 8 == 0) && (ldw % 8 == 0) && (((uintptr_t)x) % 16 == 0) &&
         (((uintptr_t)w) % 16 == 0);
}

}  // namespace vx
