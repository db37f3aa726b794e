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
#include <type_traits>

#include "common.h"

namespace vx {

typedef short v4s_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lptr_t;
// swizzle of the 16-byte pieces of a 128-byte activation row in LDS (the forward's wide kernel, gemm_wide.h)
__device__ __forceinline__ int nn_swz_x(int R) { return (R >> 1) & 7; }

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
// The same product on 256-row expert tiles x 256 output columns with the pipeline of the forward pass's wide
// kernel (gemm_wide.h): 8 wavefronts as 2 (row halves) x 4 (column quarters), a persistent walk over the
// tiles, both operands HBM/L2 -> LDS directly into two stages of 64 contraction steps, fragment reads of one
// half-step interleaved with the MFMAs of the other. The activation tile has the forward's layout (rows of
// 128 bytes, swizzled 16-byte pieces). The weight tile is 64 contraction rows x 256 columns (rows of 512
// bytes; a load instruction fills two rows), its 16-byte pieces swizzled by gb_swz for the transposing reads.
// Two products (A W + A2 W2) run as one contraction of length K + K2: the load stream switches operands at K.
// MFMA row rho of weight fragment j is output column 16 j + rho of the wavefront's 64 (a lane ends up with
// four consecutive columns per fragment). Per output element the MFMA chain is the one of the kernel above.
// Requirements (host): K, K2 multiples of 64, 32-bit byte offsets within an operand.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(512) void moe_gemm_nn_wide_kernel(MoeNnParams p, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t nw_lds[];
  constexpr int XBYTES = 256 * 64 * 2, STAGE = 2 * XBYTES;
  const int K0 = p.K[0], Ktot = K0 + (p.a[1] ? p.K[1] : 0);
  const int tiles = tiles_m * tiles_n;
  const int G = gridDim.x;  // multiple of 8
  const int first = (blockIdx.x & 7) * (G >> 3) + (blockIdx.x >> 3);
  if (first >= tiles || p.tile_group[first / tiles_n] < 0) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int wm = wave >> 2, wn = wave & 3;

  // ---- load stream: instruction q < 4 fills activation rows [8 (wave + 8 q), +8), instruction 4 + q weight rows
  // [2 (wave + 8 q), +2) of the step
  uint32_t ld_off[8];
  const bf16_t *ld_xb, *ld_wb;  // operand bases of the stream's current step (wave-uniform)
  auto uniform_ptr = [](const bf16_t* q) {
    const uint64_t v = (uint64_t)(uintptr_t)q;
    return (const bf16_t*)(uintptr_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(v >> 32)) << 32) |
                                      (uint32_t)__builtin_amdgcn_readfirstlane((int)v));
  };
  int ld_ldw = 0;
  auto set_load_tile = [&](int lin, int pair) {  // offsets and bases of operand pair `pair` on tile `lin`
    const int mt = lin / tiles_n;
    const int row0 = p.tile_row0[mt], rows = p.tile_rows[mt], n0 = (lin - mt * tiles_n) * 256;
    const int e = p.tile_group[mt];
    const int* src = pair == 0 ? p.a_src : nullptr;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int R = 8 * (wave + 8 * j) + (lane >> 3);
      const int rr = row0 + min(R, rows - 1);  // rows past the tile re-read its last row (not stored)
      const int64_t sr = src ? (int64_t)src[rr] : (int64_t)rr;
      ld_off[j] = (uint32_t)((sr * p.lda[pair] + ((lane & 7) ^ nn_swz_x(R)) * 8) * 2);
      const int Rw = 2 * (wave + 8 * j) + (lane >> 5);
      const int col = min(n0 + 8 * ((lane & 31) ^ gb_swz(Rw)), p.N - 8);  // columns past N re-read the last piece
      ld_off[4 + j] = (uint32_t)(((int64_t)Rw * p.ldw[pair] + col) * 2);
    }
    ld_ldw = __builtin_amdgcn_readfirstlane((int)p.ldw[pair]);
    ld_xb = uniform_ptr(p.a[pair]);
    ld_wb = uniform_ptr(p.w[pair] + (int64_t)e * p.w_gstride[pair]);
  };
  int ld_lin = first, ld_k = 0;
  set_load_tile(first, 0);
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)nw_lds + wave * 1024;
  // asm inside lds_load16_sv, so that the compiler does not wait for these LDS writes before unrelated fragment reads
  auto issue_one = [&](int q, int stage) {
    const uint32_t dst = lds0 + stage * STAGE + (q < 4 ? q * 8192 : XBYTES + (q - 4) * 8192);
    const bf16_t* base = q < 4 ? ld_xb : ld_wb;
    lds_load16_sv(dst, ld_off[q], base);
  };
  auto advance_loads = [&]() {  // next step of the stream; past the last tile it re-reads (unused)
    ld_k += 64;
    ld_xb += 64;
    ld_wb += 64 * ld_ldw;
    if (ld_k == K0 && Ktot > K0) set_load_tile(ld_lin, 1);
    if (ld_k >= Ktot) {
      ld_k = 0;
      const int nl = ld_lin + G;
      if (nl < tiles && p.tile_group[nl / tiles_n] >= 0) ld_lin = nl;
      set_load_tile(ld_lin, 0);
    }
  };

  f32x4 acc[8][4];  // [activation tile i][weight tile j]
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- fragment reads. Activations as in the forward kernel (k-half 1 flips bit 6). Weights: lane (r16, g)
  // addresses row 8 g + r16 / 4 (+ 4 for the upper half of the operand, + 32 for k-half 1), columns
  // 64 wn + 16 j + 4 (r16 % 4) .. + 3: 16-byte piece (8 wn + 2 j + (r16 % 4) / 2) ^ gb_swz(row), where gb_swz
  // depends on r16 / 4 and g % 2 only and 2 j meets no other term, so fragment j is the address of fragment 0
  // with 32 j flipped in.
  const int xoff = (128 * wm + r16) * 128 + ((g ^ (r16 >> 1)) * 16);
  const int wrow = 8 * g + (r16 >> 2);
  const int woff = XBYTES + wrow * 512 + (((8 * wn + ((r16 >> 1) & 1)) ^ gb_swz(wrow)) << 4) + 8 * (r16 & 1);
  struct Frag { uint4 w[4], x[8]; };
  // read number r (0 .. 15) of a fragment set: the 8 halves of the weight operands first, then the activations
  auto read_one = [&](Frag& f, int r, const uint8_t* sb, int ks) {
    if (r < 8) {
      const v4s_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) v4s_t*)(sb + ((woff ^ (32 * (r >> 1))) + (r & 1) * 2048 + ks * 16384)));
      const uint2 v2 = __builtin_bit_cast(uint2, v);
      if (r & 1) { f.w[r >> 1].z = v2.x; f.w[r >> 1].w = v2.y; }
      else { f.w[r >> 1].x = v2.x; f.w[r >> 1].y = v2.y; }
    } else {
      f.x[r - 8] = *(const uint4*)(sb + (xoff ^ (64 * ks)) + (r - 8) * 2048);
    }
  };
  // 32 MFMAs on `cur`, interleaved with the 16 reads of `nxt` and (LOADS) the global loads of a step
  auto half_step = [&](const Frag& cur, Frag& nxt, const uint8_t* nxt_sb, int nxt_ks, auto LOADS, int ld_stage) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
      for (int j = 0; j < 4; j++) acc[i][j] = mfma16(cur.w[j], cur.x[i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (decltype(LOADS)::value) {
        if (i < 4) {
          issue_one(2 * i, ld_stage);
          issue_one(2 * i + 1, ld_stage);
        }
      }
      read_one(nxt, 2 * i, nxt_sb, nxt_ks);
      read_one(nxt, 2 * i + 1, nxt_sb, nxt_ks);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  const int nk = Ktot / 64;
  Frag f0, f1;
#pragma unroll
  for (int q = 0; q < 8; q++) issue_one(q, 0);
  advance_loads();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 8; q++) issue_one(q, 1);
  advance_loads();
#pragma unroll
  for (int r = 0; r < 16; r++) read_one(f0, r, nw_lds, 0);

  int st = 0;  // stage of the current step
  for (int lin = first; lin < tiles; lin += G) {
    const int mt = lin / tiles_n;
    if (p.tile_group[mt] < 0) break;
    const int row0 = p.tile_row0[mt], rows = p.tile_rows[mt], n0 = (lin - mt * tiles_n) * 256;
    for (int kt = 0; kt < nk; kt++) {
      const uint8_t* cur_sb = nw_lds + st * STAGE;
      const uint8_t* oth_sb = nw_lds + (st ^ 1) * STAGE;
      half_step(f0, f1, cur_sb, 1, std::false_type{}, 0);
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __syncthreads();  // the next step has landed everywhere; this stage has been read by everyone
      __builtin_amdgcn_sched_barrier(0);
      half_step(f1, f0, oth_sb, 0, std::true_type{}, st);
      advance_loads();
      st ^= 1;
    }
    // lane holds C[row0 + 128 wm + 16 i + r16][n0 + 64 wn + 16 j + 4 g + c]
    const int nb = n0 + 64 * wn + 4 * g;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int m = 128 * wm + 16 * i + r16;
      bf16_t* cp = p.c + (int64_t)(row0 + m) * p.ldc + nb;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        uint2 pk;
        pk.x = pack_bf16x2(acc[i][j][0], acc[i][j][1]);
        pk.y = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
        acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (m < rows && nb + 16 * j < p.N) *(uint2*)(cp + 16 * j) = pk;
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // loads past the last step still target our LDS
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
// The same product on 256 x 256 output tiles with the pipeline of the wide kernels: 8 wavefronts as 2 (n halves
// of 128) x 4 (k quarters of 64), a persistent walk over (expert, tile) with the load stream running across
// tile boundaries, both operands HBM/L2 -> LDS directly into two stages of 64 contraction rows x 256 columns
// (rows of 512 bytes, 16-byte pieces swizzled by gb_swz; a load instruction fills two rows), transposing
// fragment reads of one half-step interleaved with the MFMAs of the other. The contraction runs over the
// expert's rows, so the lanes' load offsets change with every step: the (gathered) row numbers of a step are
// fetched one step before its loads are issued. Rows past the expert's last one are re-reads of that row, and
// are overwritten with zeros in LDS by the wavefront that loaded them before anyone reads them. Workgroup ->
// tile: an XCD (workgroup id % 8) walks runs of 32 consecutive tiles, expert-major, so an expert's rows are
// fetched into one or two L2s only. Per output element the MFMA chain is the one of the kernel above.
// Requirements (host): 32-bit byte offsets within an operand; each operand has at least one row.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(512) void moe_gemm_tn_wide_kernel(MoeTnParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t tw_lds[];
  constexpr int TBYTES = 64 * 512, STAGE = 2 * TBYTES;
  const int tiles_k = (p.K + 255) >> 8, tpe = tiles_k * ((p.N + 255) >> 8);
  const int tiles = tpe * p.E;
  const int G = gridDim.x;  // multiple of 8
  const int first = (blockIdx.x & 7) * (G >> 3) + (blockIdx.x >> 3);
  if (first >= tiles) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int wn = wave >> 2, wk = wave & 3;

  // ---- load stream. Instruction j (0 .. 3) of an operand fills tile rows Rw = 2 (wave + 8 j) + lane / 32; the
  // swizzle term gb_swz(Rw) does not depend on j, so a lane fetches the same 16-byte column piece in all four.
  const int lrow = 2 * wave + (lane >> 5);
  const int lpiece = (lane & 31) ^ gb_swz(lrow);
  int ld_lin = first, ld_s = 0, ld_lo = 0, ld_hi = 1;  // stream position: tile, step, the expert's rows
  int ld_valid = 64, landed_valid = 64;                // rows inside the expert of the next / the last issued step
  uint32_t ycol = 0, xcol = 0;                         // byte offset of this lane's column piece
  int iy[4], ix[4];                                    // row numbers of the next step to be issued
  auto tile_rows_of = [&](int lin, int& lo, int& hi) {
    const int e = lin / tpe;
    lo = p.cu[e];
    hi = p.cu[e + 1];
  };
  auto set_load_tile = [&](int lin) {
    const int t = lin % tpe;
    const int k0 = (t % tiles_k) << 8, n0 = (t / tiles_k) << 8;
    ycol = (uint32_t)(2 * min(n0 + 8 * lpiece, p.N - 8));  // columns past N / K re-read the last piece
    xcol = (uint32_t)(2 * min(k0 + 8 * lpiece, p.K - 8));
  };
  auto fetch_rows = [&]() {  // row numbers of step ld_s of the stream's tile
    ld_valid = min(64, ld_hi - ld_lo - 64 * ld_s);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int r = max(min(ld_lo + 64 * ld_s + lrow + 16 * j, ld_hi - 1), 0);
      iy[j] = p.dy_src ? p.dy_src[r] : r;
      ix[j] = p.x_src ? p.x_src[r] : r;
    }
  };
  // first tile with rows at or after `lin` (stride G); the stream stays where it is when there is none
  auto seek_tile = [&](int lin) {
    for (; lin < tiles; lin += G) {
      int lo, hi;
      tile_rows_of(lin, lo, hi);
      if (hi > lo) {
        ld_lin = lin;
        ld_lo = lo;
        ld_hi = hi;
        set_load_tile(lin);
        return;
      }
    }
  };
  seek_tile(first);
  if (ld_hi <= ld_lo) { ld_lo = 0; ld_hi = 1; set_load_tile(first); }  // nothing but experts without rows
  fetch_rows();
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)tw_lds + wave * 1024;
  uint32_t ld_off[8];
  auto set_offsets = [&]() {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      ld_off[j] = (uint32_t)iy[j] * (uint32_t)(2 * p.lddy) + ycol;
      ld_off[4 + j] = (uint32_t)ix[j] * (uint32_t)(2 * p.ldx) + xcol;
    }
    landed_valid = ld_valid;
  };
  // asm inside lds_load16_sv, so that the compiler does not wait for these LDS writes before unrelated fragment reads
  auto issue_one = [&](int q, int stage) {
    const uint32_t dst = lds0 + stage * STAGE + (q < 4 ? q * 8192 : TBYTES + (q - 4) * 8192);
    const bf16_t* base = q < 4 ? p.dy : p.x;
    lds_load16_sv(dst, ld_off[q], base);
  };
  auto advance_loads = [&]() {  // next step of the stream; past the last tile with rows it re-reads (unused)
    ld_s++;
    if (64 * ld_s >= ld_hi - ld_lo) {
      ld_s = 0;
      seek_tile(ld_lin + G);
    }
    fetch_rows();
  };
  // the wavefront's own rows of the step that has just landed in `stage`, past the expert's last row: zeros
  auto zero_tail = [&](int stage, int valid) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      if (lrow + 16 * j >= valid) {
        uint8_t* d = tw_lds + stage * STAGE + wave * 1024 + j * 8192 + lane * 16;
        *(uint4*)d = make_uint4(0u, 0u, 0u, 0u);
        *(uint4*)(d + TBYTES) = make_uint4(0u, 0u, 0u, 0u);
      }
    }
  };

  f32x4 acc[4][8];  // [k tile i][n tile f]
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int f = 0; f < 8; f++) acc[i][f] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- fragment reads: lane (r16, g) addresses row 8 g + r16 / 4 (+ 4 for the upper half of the operand, + 32
  // for the second half-step) and the 8 bytes of columns c0 + 4 (r16 % 4) .. + 3, c0 = 128 wn + 16 f (dY) or
  // 64 wk + 16 i (X): 16-byte piece (c0 / 8 + (r16 % 4) / 2) ^ gb_swz(row); 2 f and 2 i meet no other term of
  // it, so fragment f is the address of fragment 0 with 32 f flipped in.
  const int frow = 8 * g + (r16 >> 2);
  const int yoff = frow * 512 + (((16 * wn + ((r16 >> 1) & 1)) ^ gb_swz(frow)) << 4) + 8 * (r16 & 1);
  const int xoff = TBYTES + frow * 512 + (((8 * wk + ((r16 >> 1) & 1)) ^ gb_swz(frow)) << 4) + 8 * (r16 & 1);
  struct Frag { uint4 x[4], y[8]; };
  typedef __attribute__((address_space(3))) v4s_t* tr_ptr_t;
  // read number r (0 .. 23) of a fragment set: the 8 halves of the X operands first, then the 16 of dY
  auto read_one = [&](Frag& f, int r, const uint8_t* sb, int ks) {
    const int t = r < 8 ? r >> 1 : (r - 8) >> 1;
    const int off = ((r < 8 ? xoff : yoff) ^ (32 * t)) + (r & 1) * 2048 + ks * 16384;
    const uint2 v = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)(sb + off)));
    uint4& d = r < 8 ? f.x[t] : f.y[t];
    if (r & 1) { d.z = v.x; d.w = v.y; }
    else { d.x = v.x; d.y = v.y; }
  };
  // 32 MFMAs on `cur`, interleaved with the 24 reads of `nxt` and (LOADS) the global loads of a step
  auto half_step = [&](const Frag& cur, Frag& nxt, const uint8_t* nxt_sb, int nxt_ks, auto LOADS, int ld_stage) {
#pragma unroll
    for (int f = 0; f < 8; f++) {
#pragma unroll
      for (int i = 0; i < 4; i++) acc[i][f] = mfma16(cur.x[i], cur.y[f], acc[i][f]);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (decltype(LOADS)::value) {
        if (f < 4) {
          issue_one(2 * f, ld_stage);
          issue_one(2 * f + 1, ld_stage);
        }
      }
      read_one(nxt, 3 * f, nxt_sb, nxt_ks);
      read_one(nxt, 3 * f + 1, nxt_sb, nxt_ks);
      read_one(nxt, 3 * f + 2, nxt_sb, nxt_ks);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  Frag f0, f1;
  set_offsets();
#pragma unroll
  for (int q = 0; q < 8; q++) issue_one(q, 0);
  advance_loads();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (landed_valid < 64) zero_tail(0, landed_valid);
  __syncthreads();
  set_offsets();
#pragma unroll
  for (int q = 0; q < 8; q++) issue_one(q, 1);
  advance_loads();
#pragma unroll
  for (int r = 0; r < 24; r++) read_one(f0, r, tw_lds, 0);

  int st = 0;  // stage of the current step
  for (int lin = first; lin < tiles; lin += G) {
    const int e = lin / tpe, t = lin - e * tpe;
    const int k0 = (t % tiles_k) << 8, n0 = (t / tiles_k) << 8;
    const int nk = (p.cu[e + 1] - p.cu[e] + 63) >> 6;
    for (int kt = 0; kt < nk; kt++) {
      const uint8_t* cur_sb = tw_lds + st * STAGE;
      const uint8_t* oth_sb = tw_lds + (st ^ 1) * STAGE;
      half_step(f0, f1, cur_sb, 1, std::false_type{}, 0);
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      if (landed_valid < 64) zero_tail(st ^ 1, landed_valid);  // the step issued last has landed (own loads)
      __syncthreads();  // the next step is in LDS for everyone; this stage has been read by everyone
      __builtin_amdgcn_sched_barrier(0);
      set_offsets();
      half_step(f1, f0, oth_sb, 0, std::true_type{}, st);
      advance_loads();
      st ^= 1;
    }
    // lane holds dW[n0 + 128 wn + 16 f + r16][k0 + 64 wk + 16 i + 4 g + c]
    bf16_t* dwe = p.dw + (int64_t)e * p.dw_gstride;
    const int kb = k0 + 64 * wk + 4 * g;
#pragma unroll
    for (int f = 0; f < 8; f++) {
      const int n = n0 + 128 * wn + 16 * f + r16;
      bf16_t* cp = dwe + (int64_t)n * p.lddw + kb;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        uint2 pk;
        pk.x = pack_bf16x2(acc[i][f][0], acc[i][f][1]);
        pk.y = pack_bf16x2(acc[i][f][2], acc[i][f][3]);
        acc[i][f] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (n < p.N && kb + 16 * i < p.K) *(uint2*)(cp + 16 * i) = pk;
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // loads past the last step still target our LDS
}

// ---------------------------------------------------------------------------------------
// The elementwise part of the backward pass between the grouped products (fused_moe.py:150-250 of the
// reference runs it as separate bf16 tensor operations; every rounding to bf16 below stands where one of those
// operations rounds). Per sorted row r with routing weight w = rw[flat[r]], from g, u (recomputed gate / up
// projections) and d_hw (gradient of the weighted activation):
//   a = silu(g)   act = a u   hw = act w                       (the forward's values)
//   d_act = d_hw w   d_rw[flat[r]] = sum_i r16(act d_hw)   d_u = a d_act   d_g = silu'(g) (d_act u)
// One wavefront per row; the row sum runs lane-sequentially over the lane's 8-element pieces, then through the
// wavefront butterfly: the order depends on I only.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float rb(float v) { return bf16_to_f32(f32_to_bf16(v)); }

__global__ __launch_bounds__(256) void moe_swiglu_bwd_kernel(const bf16_t* __restrict__ g, const bf16_t* __restrict__ u,
                                                             const bf16_t* __restrict__ d_hw, int64_t ldg, int64_t ldu,
                                                             int64_t ldd, const bf16_t* __restrict__ rw,
                                                             const int* __restrict__ flat, bf16_t* __restrict__ hw,
                                                             bf16_t* __restrict__ d_g, bf16_t* __restrict__ d_u,
                                                             bf16_t* __restrict__ d_rw, int64_t ldh, int64_t ldog,
                                                             int64_t ldou, int64_t rows, int I) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int f = flat[r];
  const float w = bf16_to_f32(rw[f]);
  float part = 0.f;
  for (int v = lane; v < I / 8; v += 64) {
    const uint4 gv = ldg16_raw(g + r * ldg + 8 * v), uv = ldg16_raw(u + r * ldu + 8 * v), dv = ldg16_raw(d_hw + r * ldd + 8 * v);
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w}, dw[4] = {dv.x, dv.y, dv.z, dv.w};
    uint32_t oh[4], og[4], ou[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      float res[3][2];
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const float gf = h ? bf16hi(gw[j]) : bf16lo(gw[j]);
        const float uf = h ? bf16hi(uw[j]) : bf16lo(uw[j]);
        const float df = h ? bf16hi(dw[j]) : bf16lo(dw[j]);
        const float s = 1.0f / (1.0f + expf(-gf));
        const float a = rb(gf * s);
        const float act = rb(a * uf);
        const float d_act = rb(df * w);
        part += rb(act * df);
        const float d_a = rb(d_act * uf);
        res[0][h] = act * w;
        res[1][h] = d_a * s * (1.0f + gf * (1.0f - s));
        res[2][h] = a * d_act;
      }
      oh[j] = pack_bf16x2(res[0][0], res[0][1]);
      og[j] = pack_bf16x2(res[1][0], res[1][1]);
      ou[j] = pack_bf16x2(res[2][0], res[2][1]);
    }
    *(uint4*)(hw + r * ldh + 8 * v) = make_uint4(oh[0], oh[1], oh[2], oh[3]);
    *(uint4*)(d_g + r * ldog + 8 * v) = make_uint4(og[0], og[1], og[2], og[3]);
    *(uint4*)(d_u + r * ldou + 8 * v) = make_uint4(ou[0], ou[1], ou[2], ou[3]);
  }
  part = wave_sum(part);
  if (lane == 0) d_rw[f] = f32_to_bf16(part);
}

// ---------------------------------------------------------------------------------------
// Gradient of the router (softmax over E logits in fp32 -> the k selected probabilities -> optional renormalisation
// -> cast; the reference runs these as tensor operations, modeling_qwen3_moe.py:128-134) with respect to the logits:
//   p = softmax(l), sel_i = p[idx_i], (renorm) s = sum sel, w_i = sel_i / s, d_sel_i = (d_w_i - sum_j d_w_j w_j) / s,
//   d_l_j = p_j ((j == idx_i ? d_sel_i : 0) - sum_i d_sel_i sel_i).
// One wavefront per token, E <= 512, k <= 64; every sum in a fixed lane order.
// ---------------------------------------------------------------------------------------
template <bool LB, bool WB>
__global__ __launch_bounds__(256) void router_topk_bwd_kernel(const void* __restrict__ logits_, const int64_t* __restrict__ idx,
                                                              const void* __restrict__ d_w_, void* __restrict__ d_logits_,
                                                              int64_t T, int E, int k, int64_t ld, int64_t ldo, int renorm) {
  __shared__ float ps[4][512], dp[4][512];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t t_ = (int64_t)blockIdx.x * 4 + wv;
  const bool live = t_ < T;
  const int64_t t = live ? t_ : T - 1;  // a wavefront past the end recomputes the last token and stores nothing
  auto ldl = [&](int j) {
    return LB ? bf16_to_f32(((const bf16_t*)logits_)[t * ld + j]) : ((const float*)logits_)[t * ld + j];
  };
  float l[8], m = -INFINITY;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int j = lane + 64 * i;
    l[i] = j < E ? ldl(j) : -INFINITY;
    m = fmaxf(m, l[i]);
  }
  m = wave_max(m);
  float z = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    l[i] = lane + 64 * i < E ? expf(l[i] - m) : 0.f;
    z += l[i];
  }
  z = wave_sum(z);
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int j = lane + 64 * i;
    l[i] /= z;
    if (j < E) { ps[wv][j] = l[i]; dp[wv][j] = 0.f; }
  }
  __syncthreads();
  int my = -1;
  float sel = 0.f, dw = 0.f;
  if (lane < k) {
    my = (int)idx[t * k + lane];
    sel = ps[wv][my];
    dw = WB ? bf16_to_f32(((const bf16_t*)d_w_)[t * k + lane]) : ((const float*)d_w_)[t * k + lane];
  }
  float d_sel = dw;
  if (renorm) {
    const float s = wave_sum(sel);
    const float dot = wave_sum(dw * (sel / s));
    d_sel = lane < k ? (dw - dot) / s : 0.f;
  }
  const float c = wave_sum(d_sel * sel);
  if (lane < k) dp[wv][my] = d_sel;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int j = lane + 64 * i;
    if (j < E && live) {
      const float g = l[i] * (dp[wv][j] - c);
      if (LB) ((bf16_t*)d_logits_)[t * ldo + j] = f32_to_bf16(g);
      else ((float*)d_logits_)[t * ldo + j] = g;
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
                   const int* tile_rows, int64_t max_tiles, int bm, int64_t a_rows, hipStream_t stream) {
  if (!a || !w || !c || !tile_group || !tile_row0 || !tile_rows) return VX_ERR_ARG;
  if ((a2 == nullptr) != (w2 == nullptr)) return VX_ERR_ARG;
  if (N <= 0 || K <= 0 || N > 0x7fffffff || K > 0x7fffffff || max_tiles < 0) return VX_ERR_ARG;
  if (a2 && (K2 <= 0 || K2 > 0x7fffffff)) return VX_ERR_ARG;
  // a tile is at most the 128 rows one workgroup of the narrow kernel covers, or exactly the wide kernel's 256
  if (bm <= 0 || (bm > 128 && bm != 256)) return VX_ERR_UNSUPPORTED;
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
  if (bm == 256) {
    // a_rows = rows addressable in a (and a2): bounds the 32-bit load offsets
    const int64_t lim = (int64_t)1 << 32;
    if (K % 64 || (a2 && K2 % 64) || a_rows <= 0) return VX_ERR_UNSUPPORTED;
    if ((a_rows * lda + K) * 2 >= lim || (64 * ldw + N) * 2 >= lim) return VX_ERR_UNSUPPORTED;
    if (a2 && ((max_tiles * 256 * lda2 + K2) * 2 >= lim || (64 * ldw2 + N) * 2 >= lim)) return VX_ERR_UNSUPPORTED;
    const int64_t tn = (N + 255) / 256, tiles = max_tiles * tn;
    if (tiles > (1 << 30)) return VX_ERR_UNSUPPORTED;
    constexpr int LDS = 2 * 2 * 256 * 64 * 2;
    static DeviceOnce once;
    const int dev = once.slot();
    if (once.need(dev)) {
      if (hipFuncSetAttribute((const void*)moe_gemm_nn_wide_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, LDS) !=
          hipSuccess) {
        (void)hipGetLastError();
        return VX_ERR_LAUNCH;
      }
      once.mark(dev);
    }
    const unsigned grid = (unsigned)(tiles >= 256 ? 256 : (tiles + 7) / 8 * 8);
    moe_gemm_nn_wide_kernel<<<grid, 512, LDS, stream>>>(p, (int)max_tiles, (int)tn);
    return launch_status();
  }
  moe_gemm_nn_kernel<NN_ROWS><<<dim3((unsigned)((N + 127) / 128), (unsigned)max_tiles), 256, 0, stream>>>(p);
  return launch_status();
}

int vx_router_topk_bwd(const void* logits, const int64_t* idx, const void* d_weights, void* d_logits, int64_t T, int E,
                       int k, int64_t ld, int64_t ld_out, int logits_bf16, int weights_bf16, int renorm,
                       hipStream_t stream) {
  if (!logits || !idx || !d_weights || !d_logits || T < 0 || E <= 0 || k <= 0) return VX_ERR_ARG;
  if (E > 512 || k > 64 || k > E) return VX_ERR_UNSUPPORTED;
  if (T == 0) return VX_OK;
  const int64_t blocks = (T + 3) / 4;
  if (blocks > 0x7fffffffLL) return VX_ERR_ARG;
#define VX_RB(LB, WB) \
  router_topk_bwd_kernel<LB, WB><<<(unsigned)blocks, 256, 0, stream>>>(logits, idx, d_weights, d_logits, T, E, k, ld, ld_out, renorm)
  if (logits_bf16 && weights_bf16) VX_RB(true, true);
  else if (logits_bf16) VX_RB(true, false);
  else if (weights_bf16) VX_RB(false, true);
  else VX_RB(false, false);
#undef VX_RB
  return launch_status();
}

int vx_moe_swiglu_bwd(const void* g, const void* u, const void* d_hw, int64_t ldg, int64_t ldu, int64_t ldd,
                      const void* rw, const int* flat, void* hw, void* d_g, void* d_u, void* d_rw, int64_t ld_hw,
                      int64_t ld_dg, int64_t ld_du, int64_t rows, int64_t I, hipStream_t stream) {
  if (!g || !u || !d_hw || !rw || !flat || !hw || !d_g || !d_u || !d_rw) return VX_ERR_ARG;
  if (rows < 0 || I <= 0 || I > 0x7fffffff) return VX_ERR_ARG;
  if (I % 8 || ldg % 8 || ldu % 8 || ldd % 8 || ld_hw % 8 || ld_dg % 8 || ld_du % 8 || !al16(g) || !al16(u) || !al16(d_hw) || !al16(hw) || !al16(d_g) || !al16(d_u))
    return VX_ERR_UNSUPPORTED;
  if (rows == 0) return VX_OK;
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffffLL) return VX_ERR_UNSUPPORTED;
  moe_swiglu_bwd_kernel<<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)g, (const bf16_t*)u, (const bf16_t*)d_hw, ldg,
                                                              ldu, ldd, (const bf16_t*)rw, flat, (bf16_t*)hw, (bf16_t*)d_g,
                                                              (bf16_t*)d_u, (bf16_t*)d_rw, ld_hw, ld_dg, ld_du, rows, (int)I);
  return launch_status();
}

int vx_moe_gemm_tn(const void* dy, int64_t lddy, const int* dy_src, const void* x, int64_t ldx, const int* x_src,
                   void* dw, int64_t lddw, int64_t dw_gstride, int64_t N, int64_t K, const int* cu, int64_t num_experts,
                   int64_t dy_rows, int64_t x_rows, hipStream_t stream) {
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
  // dy_rows / x_rows = rows addressable in dy / x: the wide kernel's 32-bit offsets must reach them
  const int64_t lim = (int64_t)1 << 32;
  const int64_t tiles = num_experts * ((K + 255) / 256) * ((N + 255) / 256);
  if (N >= 256 && K >= 256 && dy_rows > 0 && x_rows > 0 && (dy_rows * lddy + N) * 2 < lim &&
      (x_rows * ldx + K) * 2 < lim && tiles <= (1 << 30)) {
    constexpr int LDS = 2 * 2 * 64 * 512;
    static DeviceOnce once;
    const int dev = once.slot();
    if (once.need(dev)) {
      if (hipFuncSetAttribute((const void*)moe_gemm_tn_wide_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, LDS) !=
          hipSuccess) {
        (void)hipGetLastError();
        return VX_ERR_LAUNCH;
      }
      once.mark(dev);
    }
    const unsigned grid = (unsigned)(tiles >= 256 ? 256 : (tiles + 7) / 8 * 8);
    moe_gemm_tn_wide_kernel<<<grid, 512, LDS, stream>>>(p);
  } else {
    moe_gemm_tn_kernel<TN_ROWS><<<dim3((unsigned)((K + 127) / 128), (unsigned)gy, (unsigned)num_experts), 256, 0, stream>>>(p);
  }
  return launch_status();
}

}  // extern "C"
