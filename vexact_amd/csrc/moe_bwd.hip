// Grouped matrix products of the fused-MoE backward pass (the reference computes them with its Triton
// group GEMMs, vexact/batch_invariant_ops/fused_moe.py:126-265):
//   * vx_moe_gemm_nn: C[rows of expert e] = A[rows of e] W_e (+ A2[rows of e] W2_e), W_e = [K, N] with N
//     contiguous. This is the data gradient of a projection whose weight is stored [out = K, in = N].
//   * vx_moe_gemm_tn: dW_e [N, K] = sum over the rows r of expert e of dY[r, :]^T X[r, :], the weight gradient.
// In both the contraction index is the slow index of a row-major operand. Such an operand is staged in LDS
// as a tile of 32 or 64 rows x 128 columns and read with transposing reads (ds_read_b64_tr_b16): the 16 lanes of
// a group address 4 rows x 16 columns in 8-byte pieces and each lane receives one column of those 4 rows,
// which is the MFMA operand layout (lane (r16, g): index r16, contraction slots 8 g .. 8 g + 7).
// Every output element is one ascending chain of MFMAs over its expert's rows (or over K), with no atomics
// and no split of the contraction, so results do not depend on the launch shape or on other experts.
#include "common.h"

namespace vx {

typedef short v4s_t __attribute__((ext_vector_type(4)));

// An LDS tile holds GB_ROWS contraction rows (a multiple of the 32 of one MFMA) of 128 bf16.
constexpr int NN_ROWS = 64;  // per k-step of the data-gradient kernel (its LDS use is one operand only)
constexpr int TN_ROWS = 32;  // of the weight-gradient kernel: measured faster than 64 (more workgroups per CU, shorter ragged tails)

// A transposing read takes two adjacent 16-byte pieces from each of the rows 8 g .. 8 g + 3 (or + 4 .. + 7) of
// two lane groups g at a time: 16-byte piece c of row r lives at piece c ^ gb_swz(r), whose pair index
// differs over those eight rows, so they fall into different banks
__device__ __forceinline__ int gb_swz(int row) { return ((row & 3) | ((row >> 1) & 4)) << 1; }
__device__ __forceinline__ int gb_off(int row, int byte) {
  return row * 256 + ((((byte >> 4) ^ gb_swz(row)) << 4) | (byte & 15));
}

// columns col0 .. col0 + 15, rows row0 .. row0 + 31 of the tile as an MFMA operand: lane (r16, g) gets column
// col0 + r16, rows row0 + 8 g .. row0 + 8 g + 7
__device__ __forceinline__ uint4 gb_frag(const uint8_t* tile, int row0, int col0, int r16, int g) {
  const int byte = 2 * col0 + 8 * (r16 & 3);
  const int row_lo = row0 + 8 * g + (r16 >> 2), row_hi = row_lo + 4;
  const v4s_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s_t*)(tile + gb_off(row_lo, byte)));
  const v4s_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s_t*)(tile + gb_off(row_hi, byte)));
  const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
  return make_uint4(lo2.x, lo2.y, hi2.x, hi2.y);
}

// ---------------------------------------------------------------------------------------
// C = A W (+ A2 W2) per expert tile of up to 128 rows; 128 output columns per workgroup; 4 wavefronts
// as 2 (row halves) x 2 (column halves), each 64 x 64 = 4 x 4 MFMA tiles. The activation operand is
// loaded from global memory in operand form (16 bytes per lane, like the forward kernels).
// ---------------------------------------------------------------------------------------
struct MoeNnParams {
  const bf16_t* a[2];
  int64_t lda[2];
  const bf16_t* w[2];
  int64_t ldw[2], w_gstride[2];
  int K[2];
  const int* a_src;  // optional: row r of a[0] is a[0][a_src[r]]
  bf16_t* c;
  int64_t ldc;
  int N;
  const int *tile_group, *tile_row0, *tile_rows;
};

template <int GB_ROWS>
__global__ __launch_bounds__(256) void moe_gemm_nn_kernel(MoeNnParams p) {
  constexpr int GB_PIECES = GB_ROWS * 16 / 256, GB_TILE = GB_ROWS * 256;  // 16-byte pieces per thread; bytes
  __shared__ __attribute__((aligned(1024))) uint8_t wt[2][GB_TILE];
  const int t = blockIdx.y;
  const int e = p.tile_group[t];
  if (e < 0) return;  // uniform over the block
  const int row0 = p.tile_row0[t], rows = p.tile_rows[t];
  if (rows <= 0) return;
  const int n0 = blockIdx.x * 128;
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int wave = threadIdx.x >> 6, wr = wave >> 1, wn = wave & 1;

  f32x4 acc[4][4];
#pragma unroll
  for (int rt = 0; rt < 4; rt++)
#pragma unroll
    for (int f = 0; f < 4; f++) acc[rt][f] = f32x4{0.f, 0.f, 0.f, 0.f};

  int buf = 0;
#pragma unroll 1
  for (int pair = 0; pair < 2; pair++) {
    const bf16_t* a = p.a[pair];
    if (!a) break;  // uniform
    const int K = p.K[pair];
    const int64_t lda = p.lda[pair], ldw = p.ldw[pair];
    const bf16_t* w = p.w[pair] + (int64_t)e * p.w_gstride[pair];
    // activation rows of this lane's four row tiles (rows past the tile read its last row; never stored)
    const bf16_t* ap[4];
#pragma unroll
    for (int rt = 0; rt < 4; rt++) {
      int r = row0 + min(64 * wr + 16 * rt + r16, rows - 1);
      if (pair == 0 && p.a_src) r = p.a_src[r];
      ap[rt] = a + (int64_t)r * lda + 8 * g;
    }
    // this thread's two 16-byte pieces of a weight tile: piece q = tid + 256 j -> row q / 16, piece q % 16
    // A step that lies fully inside K (and a column tile fully inside N) is loaded without masks: the masks
    // cost four selects per load, as many vector instructions as the products they feed.
    const bool full_n = n0 + 128 <= p.N;  // uniform
    auto load_w = [&](int k0, uint4 (&wreg)[GB_PIECES]) {
      if (full_n && k0 + GB_ROWS <= K) {
#pragma unroll
        for (int j = 0; j < GB_PIECES; j++) {
          const int q = threadIdx.x + 256 * j;
          wreg[j] = ldg16_raw(w + (int64_t)(k0 + (q >> 4)) * ldw + n0 + 8 * (q & 15));
        }
      } else {
#pragma unroll
        for (int j = 0; j < GB_PIECES; j++) {
          const int q = threadIdx.x + 256 * j, row = q >> 4, pc = q & 15;
          const bool ok = k0 + row < K && n0 + 8 * pc < p.N;
          wreg[j] = ldg16(ok ? (const void*)(w + (int64_t)(k0 + row) * ldw + n0 + 8 * pc) : (const void*)w, ok);
        }
      }
    };
    auto load_a = [&](int k0, uint4 (&af)[GB_ROWS / 32][4]) {
      if (k0 + GB_ROWS <= K) {
#pragma unroll
        for (int kc = 0; kc < GB_ROWS / 32; kc++)
#pragma unroll
          for (int rt = 0; rt < 4; rt++) af[kc][rt] = ldg16_raw(ap[rt] + k0 + 32 * kc);
      } else {
#pragma unroll
        for (int kc = 0; kc < GB_ROWS / 32; kc++) {
          const bool ok = k0 + 32 * kc + 8 * g < K;
#pragma unroll
          for (int rt = 0; rt < 4; rt++) af[kc][rt] = ldg16(ok ? ap[rt] + k0 + 32 * kc : a, ok);
        }
      }
    };
    const int steps = (K + GB_ROWS - 1) / GB_ROWS;
    uint4 wreg[GB_PIECES], af[GB_ROWS / 32][4];
    load_w(0, wreg);
    load_a(0, af);
#pragma unroll 1
    for (int s = 0; s < steps; s++) {
#pragma unroll
      for (int j = 0; j < GB_PIECES; j++) {
        const int q = threadIdx.x + 256 * j;
        *(uint4*)(wt[buf] + gb_off(q >> 4, 16 * (q & 15))) = wreg[j];
      }
      __syncthreads();  // also: everyone is done reading the other buffer's previous contents
      uint4 afn[GB_ROWS / 32][4];
      if (s + 1 < steps) {
        load_w((s + 1) * GB_ROWS, wreg);
        load_a((s + 1) * GB_ROWS, afn);
      }
#pragma unroll
      for (int kc = 0; kc < GB_ROWS / 32; kc++) {
        uint4 wf[4];
#pragma unroll
        for (int f = 0; f < 4; f++) wf[f] = gb_frag(wt[buf], 32 * kc, 64 * wn + 16 * f, r16, g);
#pragma unroll
        for (int rt = 0; rt < 4; rt++)
#pragma unroll
          for (int f = 0; f < 4; f++) acc[rt][f] = mfma16(wf[f], af[kc][rt], acc[rt][f]);
      }
      if (s + 1 < steps) {
#pragma unroll
        for (int kc = 0; kc < GB_ROWS / 32; kc++)
#pragma unroll
          for (int rt = 0; rt < 4; rt++) af[kc][rt] = afn[kc][rt];
      }
      buf ^= 1;
    }
  }

  // lane (r16, g) holds, for row tile rt and column tile f, row r16 and columns 4 g .. 4 g + 3
#pragma unroll
  for (int rt = 0; rt < 4; rt++) {
    const int lr = 64 * wr + 16 * rt + r16;
    if (lr >= rows) continue;
    bf16_t* cp = p.c + (int64_t)(row0 + lr) * p.ldc;
#pragma unroll
    for (int f = 0; f < 4; f++) {
      const int n = n0 + 64 * wn + 16 * f + 4 * g;
      if (n >= p.N) continue;
      uint2 pk;
      pk.x = pack_bf16x2(acc[rt][f][0], acc[rt][f][1]);
      pk.y = pack_bf16x2(acc[rt][f][2], acc[rt][f][3]);
      *(uint2*)(cp + n) = pk;
    }
  }
}

// ---------------------------------------------------------------------------------------
// dW_e[n][k] = sum_r dY[r][n] X[r][k] over the sorted rows cu[e] <= r < cu[e + 1]; one workgroup per
// (expert, 128 x 128 output tile); both operands go through LDS tiles of 32 rows. Experts without rows
// get zeros.
// ---------------------------------------------------------------------------------------
struct MoeTnParams {
  const bf16_t* dy;
  int64_t lddy;
  const int* dy_src;  // optional row gathers: row r of an operand is operand[src[r]]
  const bf16_t* x;
  int64_t ldx;
  const int* x_src;
  bf16_t* dw;
  int64_t lddw, dw_gstride;
  int N, K, E;
  const int* cu;
};

template <int GB_ROWS>
__global__ __launch_bounds__(256) void moe_gemm_tn_kernel(MoeTnParams p) {
  constexpr int GB_PIECES = GB_ROWS * 16 / 256, GB_TILE = GB_ROWS * 256;
  __shared__ __attribute__((aligned(1024))) uint8_t yt[2][GB_TILE];
  __shared__ __attribute__((aligned(1024))) uint8_t xt[2][GB_TILE];
  const int e = blockIdx.z;
  const int lo = p.cu[e], hi = p.cu[e + 1];
  const int k0 = blockIdx.x * 128, n0 = blockIdx.y * 128;
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int wave = threadIdx.x >> 6, wn = wave >> 1, wk = wave & 1;

  f32x4 acc[4][4];  // [k tile][n tile]
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int f = 0; f < 4; f++) acc[i][f] = f32x4{0.f, 0.f, 0.f, 0.f};

  // piece q = tid + 256 j of a tile: row q / 16, 16-byte piece q % 16
  auto load_tiles = [&](int r0, uint4 (&yr)[GB_PIECES], uint4 (&xr)[GB_PIECES]) {
#pragma unroll
    for (int j = 0; j < GB_PIECES; j++) {
      const int q = threadIdx.x + 256 * j, row = q >> 4, pc = q & 15;
      const int r = r0 + row;
      const bool ok = r < hi;
      const int ry = ok ? (p.dy_src ? p.dy_src[r] : r) : 0;
      const int rx = ok ? (p.x_src ? p.x_src[r] : r) : 0;
      const bool oky = ok && n0 + 8 * pc < p.N, okx = ok && k0 + 8 * pc < p.K;
      yr[j] = ldg16(oky ? (const void*)(p.dy + (int64_t)ry * p.lddy + n0 + 8 * pc) : (const void*)p.dy, oky);
      xr[j] = ldg16(okx ? (const void*)(p.x + (int64_t)rx * p.ldx + k0 + 8 * pc) : (const void*)p.x, okx);
    }
  };

  const int steps = (hi - lo + GB_ROWS - 1) / GB_ROWS;
  uint4 yr[GB_PIECES], xr[GB_PIECES];
  if (steps > 0) load_tiles(lo, yr, xr);
  int buf = 0;
#pragma unroll 1
  for (int s = 0; s < steps; s++) {
#pragma unroll
    for (int j = 0; j < GB_PIECES; j++) {
      const int q = threadIdx.x + 256 * j;
      const int off = gb_off(q >> 4, 16 * (q & 15));
      *(uint4*)(yt[buf] + off) = yr[j];
      *(uint4*)(xt[buf] + off) = xr[j];
    }
    __syncthreads();
    if (s + 1 < steps) load_tiles(lo + (s + 1) * GB_ROWS, yr, xr);
#pragma unroll
    for (int kc = 0; kc < GB_ROWS / 32; kc++) {
      uint4 yf[4], xf[4];
#pragma unroll
      for (int f = 0; f < 4; f++) {
        yf[f] = gb_frag(yt[buf], 32 * kc, 64 * wn + 16 * f, r16, g);
        xf[f] = gb_frag(xt[buf], 32 * kc, 64 * wk + 16 * f, r16, g);
      }
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int f = 0; f < 4; f++) acc[i][f] = mfma16(xf[i], yf[f], acc[i][f]);
    }
    buf ^= 1;
  }

  // lane (r16, g) holds, for k tile i and n tile f, output row n = r16 and columns k = 4 g .. 4 g + 3
  bf16_t* dwe = p.dw + (int64_t)e * p.dw_gstride;
#pragma unroll
  for (int f = 0; f < 4; f++) {
    const int n = n0 + 64 * wn + 16 * f + r16;
    if (n >= p.N) continue;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int k = k0 + 64 * wk + 16 * i + 4 * g;
      if (k >= p.K) continue;
      uint2 pk;
      pk.x = pack_bf16x2(acc[i][f][0], acc[i][f][1]);
      pk.y = pack_bf16x2(acc[i][f][2], acc[i][f][3]);
      *(uint2*)(dwe + (int64_t)n * p.lddw + k) = pk;
    }
  }
}

// ---------------------------------------------------------------------------------------
// The same product on 256 x 256 output tiles: 8 wavefronts as 2 (n halves of 128) x 4 (k quarters of 64),
// LDS tiles of 32 rows x 256 columns (512-byte rows). Half the operand traffic per output element of the
// 128 x 128 kernel, which is what bounds that one; two steps of global loads are in flight in registers
// because only one workgroup fits a CU.
// ---------------------------------------------------------------------------------------
constexpr int TW_ROWS = 32, TW_TILE = TW_ROWS * 512;

__device__ __forceinline__ int tw_off(int row, int byte) {
  return row * 512 + ((((byte >> 4) ^ gb_swz(row)) << 4) | (byte & 15));
}
__device__ __forceinline__ uint4 tw_frag(const uint8_t* tile, int col0, int r16, int g) {
  const int byte = 2 * col0 + 8 * (r16 & 3);
  const int row_lo = 8 * g + (r16 >> 2), row_hi = row_lo + 4;
  const v4s_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s_t*)(tile + tw_off(row_lo, byte)));
  const v4s_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s_t*)(tile + tw_off(row_hi, byte)));
  const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
  return make_uint4(lo2.x, lo2.y, hi2.x, hi2.y);
}

__global__ __launch_bounds__(512) void moe_gemm_tn_wide_kernel(MoeTnParams p) {
  __shared__ __attribute__((aligned(1024))) uint8_t yt[2][TW_TILE];
  __shared__ __attribute__((aligned(1024))) uint8_t xt[2][TW_TILE];
  // Consecutive workgroup ids go to different XCDs (id % 8), each with its own L2: XCD x takes the experts
  // e = x (mod 8), all output tiles of one expert in a row, so an expert's rows are fetched into one L2.
  const int tiles_k = (p.K + 255) >> 8, tiles = tiles_k * ((p.N + 255) >> 8);
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int e = (slot / tiles) * 8 + xcd;
  if (e >= p.E) return;  // uniform
  const int tile = slot % tiles;
  const int lo = p.cu[e], hi = p.cu[e + 1];
  const int k0 = (tile % tiles_k) * 256, n0 = (tile / tiles_k) * 256;
  const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
  const int wave = threadIdx.x >> 6, wn = wave >> 2, wk = wave & 3;

  f32x4 acc[4][8];  // [k tile][n tile]
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int f = 0; f < 8; f++) acc[i][f] = f32x4{0.f, 0.f, 0.f, 0.f};

  // piece q = tid + 512 j of a tile: row q / 32, 16-byte piece q % 32. The (gathered) row numbers of a
  // step are fetched one step before its data, so that the two dependent loads do not add their latencies.
  auto load_rows = [&](int r0, int (&ry)[2], int (&rx)[2]) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int r = r0 + ((threadIdx.x + 512 * j) >> 5);
      const bool ok = r < hi;
      ry[j] = ok ? (p.dy_src ? p.dy_src[r] : r) : -1;
      rx[j] = ok ? (p.x_src ? p.x_src[r] : r) : -1;
    }
  };
  // `full` (uniform): every row of the step exists and the output tile lies inside N x K: no masks
  const bool full_nk = n0 + 256 <= p.N && k0 + 256 <= p.K;
  auto load_tiles = [&](bool full, const int (&ry)[2], const int (&rx)[2], uint4 (&yr)[2], uint4 (&xr)[2]) {
    if (full) {
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int pc = (threadIdx.x + 512 * j) & 31;
        yr[j] = ldg16_raw(p.dy + (int64_t)ry[j] * p.lddy + n0 + 8 * pc);
        xr[j] = ldg16_raw(p.x + (int64_t)rx[j] * p.ldx + k0 + 8 * pc);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int pc = (threadIdx.x + 512 * j) & 31;
        const bool oky = ry[j] >= 0 && n0 + 8 * pc < p.N, okx = rx[j] >= 0 && k0 + 8 * pc < p.K;
        yr[j] = ldg16(oky ? (const void*)(p.dy + (int64_t)ry[j] * p.lddy + n0 + 8 * pc) : (const void*)p.dy, oky);
        xr[j] = ldg16(okx ? (const void*)(p.x + (int64_t)rx[j] * p.ldx + k0 + 8 * pc) : (const void*)p.x, okx);
      }
    }
  };

  const int steps = (hi - lo + TW_ROWS - 1) / TW_ROWS;
  uint4 yr[2][2], xr[2][2];  // register set (s & 1) holds step s
  int ry[2], rx[2];          // row numbers of the next step to be loaded
  load_rows(lo, ry, rx);
  if (steps > 0) load_tiles(full_nk && lo + TW_ROWS <= hi, ry, rx, yr[0], xr[0]);
  load_rows(lo + TW_ROWS, ry, rx);
  if (steps > 1) load_tiles(full_nk && lo + 2 * TW_ROWS <= hi, ry, rx, yr[1], xr[1]);
  load_rows(lo + 2 * TW_ROWS, ry, rx);
  auto step = [&](int s, int buf, uint4 (&yrs)[2], uint4 (&xrs)[2]) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int q = threadIdx.x + 512 * j;
      const int off = tw_off(q >> 5, 16 * (q & 31));
      *(uint4*)(yt[buf] + off) = yrs[j];
      *(uint4*)(xt[buf] + off) = xrs[j];
    }
    __syncthreads();  // also: everyone is done reading the other buffer's previous contents
    if (s + 2 < steps) {
      load_tiles(full_nk && lo + (s + 3) * TW_ROWS <= hi, ry, rx, yrs, xrs);
      load_rows(lo + (s + 3) * TW_ROWS, ry, rx);
    }
    uint4 yf[8], xf[4];
#pragma unroll
    for (int f = 0; f < 8; f++) yf[f] = tw_frag(yt[buf], 128 * wn + 16 * f, r16, g);
#pragma unroll
    for (int i = 0; i < 4; i++) xf[i] = tw_frag(xt[buf], 64 * wk + 16 * i, r16, g);
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int f = 0; f < 8; f++) acc[i][f] = mfma16(xf[i], yf[f], acc[i][f]);
  };
#pragma unroll 1
  for (int s = 0; s < steps; s += 2) {
    step(s, 0, yr[0], xr[0]);
    if (s + 1 < steps) step(s + 1, 1, yr[1], xr[1]);
  }

  bf16_t* dwe = p.dw + (int64_t)e * p.dw_gstride;
#pragma unroll
  for (int f = 0; f < 8; f++) {
    const int n = n0 + 128 * wn + 16 * f + r16;
    if (n >= p.N) continue;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int k = k0 + 64 * wk + 16 * i + 4 * g;
      if (k >= p.K) continue;
      uint2 pk;
      pk.x = pack_bf16x2(acc[i][f][0], acc[i][f][1]);
      pk.y = pack_bf16x2(acc[i][f][2], acc[i][f][3]);
      *(uint2*)(dwe + (int64_t)n * p.lddw + k) = pk;
    }
  }
}

static inline bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace vx

using namespace vx;

extern "C" {

int vx_moe_gemm_nn(const void* a, int64_t lda, const int* a_src, const void* w, int64_t ldw, int64_t w_gstride,
                   int64_t K, const void* a2, int64_t lda2, const void* w2, int64_t ldw2, int64_t w2_gstride,
                   int64_t K2, void* c, int64_t ldc, int64_t N, const int* tile_group, const int* tile_row0,
                   const int* tile_rows, int64_t max_tiles, int bm, hipStream_t stream) {
  if (!a || !w || !c || !tile_group || !tile_row0 || !tile_rows) return VX_ERR_ARG;
  if ((a2 == nullptr) != (w2 == nullptr)) return VX_ERR_ARG;
  if (N <= 0 || K <= 0 || N > 0x7fffffff || K > 0x7fffffff || max_tiles < 0) return VX_ERR_ARG;
  if (a2 && (K2 <= 0 || K2 > 0x7fffffff)) return VX_ERR_ARG;
  if (bm <= 0 || bm > 128) return VX_ERR_UNSUPPORTED;  // a tile is at most the 128 rows one workgroup covers
  if (N % 8 || K % 8 || lda % 8 || ldw % 8 || w_gstride % 8 || ldc % 4 || !al16(a) || !al16(w) || ((uintptr_t)c & 7))
    return VX_ERR_UNSUPPORTED;
  if (a2 && (K2 % 8 || lda2 % 8 || ldw2 % 8 || w2_gstride % 8 || !al16(a2) || !al16(w2))) return VX_ERR_UNSUPPORTED;
  if (max_tiles == 0) return VX_OK;
  if (max_tiles > 65535) return VX_ERR_UNSUPPORTED;
  MoeNnParams p = {};
  p.a[0] = (const bf16_t*)a; p.lda[0] = lda; p.w[0] = (const bf16_t*)w; p.ldw[0] = ldw; p.w_gstride[0] = w_gstride;
  p.K[0] = (int)K;
  p.a[1] = (const bf16_t*)a2; p.lda[1] = lda2; p.w[1] = (const bf16_t*)w2; p.ldw[1] = ldw2; p.w_gstride[1] = w2_gstride;
  p.K[1] = (int)K2;
  p.a_src = a_src;
  p.c = (bf16_t*)c; p.ldc = ldc; p.N = (int)N;
  p.tile_group = tile_group; p.tile_row0 = tile_row0; p.tile_rows = tile_rows;
  moe_gemm_nn_kernel<NN_ROWS><<<dim3((unsigned)((N + 127) / 128), (unsigned)max_tiles), 256, 0, stream>>>(p);
  return launch_status();
}

int vx_moe_gemm_tn(const void* dy, int64_t lddy, const int* dy_src, const void* x, int64_t ldx, const int* x_src,
                   void* dw, int64_t lddw, int64_t dw_gstride, int64_t N, int64_t K, const int* cu, int64_t num_experts,
                   hipStream_t stream) {
  if (!dy || !x || !dw || !cu) return VX_ERR_ARG;
  if (N <= 0 || K <= 0 || N > 0x7fffffff || K > 0x7fffffff || num_experts < 0) return VX_ERR_ARG;
  if (N % 8 || K % 8 || lddy % 8 || ldx % 8 || lddw % 4 || dw_gstride % 4 || !al16(dy) || !al16(x) || ((uintptr_t)dw & 7))
    return VX_ERR_UNSUPPORTED;
  if (num_experts == 0) return VX_OK;
  const int64_t gy = (N + 127) / 128;
  if (num_experts > 65535 || gy > 65535) return VX_ERR_UNSUPPORTED;
  MoeTnParams p = {};
  p.dy = (const bf16_t*)dy; p.lddy = lddy; p.dy_src = dy_src;
  p.x = (const bf16_t*)x; p.ldx = ldx; p.x_src = x_src;
  p.dw = (bf16_t*)dw; p.lddw = lddw; p.dw_gstride = dw_gstride;
  p.N = (int)N; p.K = (int)K; p.E = (int)num_experts; p.cu = cu;
  if (N >= 256 && K >= 256) {
    const int64_t wg = 8 * ((num_experts + 7) / 8) * ((K + 255) / 256) * ((N + 255) / 256);
    if (wg > 0x7fffffffLL) return VX_ERR_UNSUPPORTED;
    moe_gemm_tn_wide_kernel<<<dim3((unsigned)wg), 512, 0, stream>>>(p);
  } else {
    moe_gemm_tn_kernel<TN_ROWS><<<dim3((unsigned)((K + 127) / 128), (unsigned)gy, (unsigned)num_experts), 256, 0, stream>>>(p);
  }
  return launch_status();
}

}  // extern "C"
