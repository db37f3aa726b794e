// Wide-tile bf16 "NT" GEMM for many rows (prefill): C[m, n] = r16(sum_k X[m, k] W[n, k] (+ bias[n])).
//
// One workgroup = 8 wavefronts (two per SIMD) computes 256 (activation rows) x 256 (weight rows)
// tiles, 64 k-elements per step, and walks over several tiles (persistent). Both operand tiles go
// HBM/L2 -> LDS directly (global_load_lds_dwordx4: a wavefront writes 1 KB = 8 tile rows of 128
// bytes per instruction, no staging registers, no ds_write) into two stages of 64 KB. The 16-byte
// pieces of a tile row are stored XOR-swizzled - the lane that fills slot s of row R fetches logical
// piece s ^ swz(R) - so the 16 rows x 16 bytes of one MFMA fragment read hit 64 distinct banks
// although the rows are unpadded.
//
// Wavefront (wm, wn) of the 2 x 4 arrangement owns activation rows [128 wm, +128) and weight rows
// [64 wn, +64): 8 x 4 MFMA tiles, 12 fragment reads per 32 MFMAs. MFMA row rho of weight fragment j
// is weight row 16 (rho / 4) + 4 j + rho % 4 of the wavefront's 64, which makes a lane's 16 outputs
// of one activation row contiguous in n: the epilogue writes 16-byte pieces, 128 bytes per row.
//
// Pipeline per step: [32 MFMAs on k-half 0 | reads of k-half 1] barrier [32 MFMAs on k-half 1 |
// global loads of step + 2 into the stage just released | reads of k-half 0 of step + 1]. The load
// stream runs across tile boundaries, so the first two steps of the next tile are already on their
// way while the epilogue of the current one stores.
//
// Arithmetic per output element is the same as in the other GEMM kernels (A = weight fragment,
// B = activation fragment, K ascending in 32-chunks), so results are bit-identical to theirs.
// Requirements (checked by the host): K % 64 == 0, 16-byte aligned rows, operands below 4 GiB. Rows
// past M / N are clamped on load (a C row depends only on its own X row, a column only on its own W
// row) and masked on store.
//
// Workgroup -> tile mapping: consecutive workgroup ids go to different XCDs (id % 8), each with its
// own L2, so the ids are regrouped such that one XCD works on a contiguous run of tiles, and tiles are
// ordered in panels of 4 row tiles x all column tiles: the ~32 tiles in flight on an XCD then share
// 4 activation panels and 8 weight panels.
#pragma once
#include <type_traits>

#include "gemm_core.h"

namespace vx {

constexpr int WD_BM = 256, WD_BN = 256, WD_BK = 64;
constexpr int WD_XBYTES = WD_BM * WD_BK * 2;             // 32 KB
constexpr int WD_STAGE = (WD_BM + WD_BN) * WD_BK * 2;    // 64 KB
constexpr int WD_LDS = 2 * WD_STAGE;                     // 128 KB
constexpr int WD_GROUP_M = 4;

typedef __attribute__((address_space(3))) void* lptr_t;

__device__ __forceinline__ int wd_swz_x(int R) { return (R >> 1) & 7; }
__device__ __forceinline__ int wd_swz_w(int R) { return (((R >> 4) & 3) << 1) | ((R >> 1) & 1); }

__global__ __launch_bounds__(512) void gemm_wide_kernel(GemmParams p, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t wd_lds[];

  const int M = p.M, N = p.N, K = p.K;
  const int tiles = tiles_m * tiles_n;
  const int G = gridDim.x;  // multiple of 8
  const int first = (blockIdx.x & 7) * (G >> 3) + (blockIdx.x >> 3);
  if (first >= tiles) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int wm = wave >> 2, wn = wave & 3;

  auto tile_origin = [&](int lin, int& row0, int& n0) {
    const int span = WD_GROUP_M * tiles_n;
    const int grp = lin / span;
    const int gm0 = grp * WD_GROUP_M;
    const int gsz = min(WD_GROUP_M, tiles_m - gm0);
    const int rem = lin - grp * span;
    row0 = (gm0 + rem % gsz) * WD_BM;
    n0 = (rem / gsz) * WD_BN;
  };

  // ---- load stream: instruction q of a step fills tile rows [8 (wave + 8 (q & 3)), +8) of X (q < 4)
  // or W (q >= 4). Byte offsets from the operand base fit 32 bits (host check).
  const int lrow = lane >> 3, lslot = lane & 7;
  uint32_t ld_off[8];
  auto set_load_tile = [&](int lin) {
    int row0, n0;
    tile_origin(lin, row0, n0);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int R = 8 * (wave + 8 * j) + lrow;
      ld_off[j] = (uint32_t)(((int64_t)min(row0 + R, M - 1) * p.ldx + (lslot ^ wd_swz_x(R)) * 8) * 2);
      ld_off[4 + j] = (uint32_t)(((int64_t)min(n0 + R, N - 1) * p.ldw + (lslot ^ wd_swz_w(R)) * 8) * 2);
    }
  };
  int ld_lin = first, ld_k = 0;
  set_load_tile(ld_lin);
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)wd_lds + wave * 1024;
  // The loads are written as asm so that the compiler does not track them: told that they write LDS,
  // it would wait for them (vmcnt(0)) before the first fragment read after they are issued. The
  // wait that matters is the explicit one before the barrier that precedes their first use.
  auto issue_one = [&](int q, int stage) {
    const uint32_t dst = lds0 + stage * WD_STAGE + (q >> 2) * WD_XBYTES + (q & 3) * 8192;
    const bf16_t* base = (q < 4 ? p.x : p.w) + ld_k;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(dst), "v"(ld_off[q]), "s"(base) : "memory", "m0");
  };
  auto advance_loads = [&]() {  // next step of the stream; past the last tile it re-reads (unused)
    ld_k += WD_BK;
    if (ld_k >= K) {
      ld_k = 0;
      if (ld_lin + G < tiles) {
        ld_lin += G;
        set_load_tile(ld_lin);
      }
    }
  };

  f32x4 acc[8][4];  // [activation tile i][weight tile j]
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- fragment reads, k-half 0; k-half 1 is the same address with bit 6 flipped (slot ^ 4).
  // Activation rows 128 wm + 16 i + r16: swizzle term r16 >> 1. Weight rows
  // 64 wn + 16 (r16 / 4) + 4 j + r16 % 4: swizzle term 2 (r16 / 4) + (r16 % 4) / 2.
  const int xoff = (128 * wm + r16) * 128 + ((g ^ (r16 >> 1)) * 16);
  const int woff = WD_XBYTES + (64 * wn + 16 * (r16 >> 2) + (r16 & 3)) * 128 +
                   ((g ^ (((r16 >> 2) << 1) | ((r16 >> 1) & 1))) * 16);
  struct Frag { uint4 w[4], x[8]; };
  // read number r (0..11) of a fragment set: the 4 weight operands first, then the 8 activation ones
  auto read_one = [&](Frag& f, int r, const uint8_t* sb, int ks) {
    if (r < 4) f.w[r] = *(const uint4*)(sb + (woff ^ (64 * ks)) + r * 512);
    else f.x[r - 4] = *(const uint4*)(sb + (xoff ^ (64 * ks)) + (r - 4) * 2048);
  };
  // 32 MFMAs on `cur`, interleaved with the 12 reads of `nxt` and (LOADS) the 8 global loads of a step
  auto half_step = [&](const Frag& cur, Frag& nxt, const uint8_t* nxt_sb, int nxt_ks, auto LOADS,
                       int ld_stage) {
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
      if (i < 4) {
        read_one(nxt, 2 * i, nxt_sb, nxt_ks);
        read_one(nxt, 2 * i + 1, nxt_sb, nxt_ks);
      } else {
        read_one(nxt, 4 + i, nxt_sb, nxt_ks);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  const int nk = K / WD_BK;
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
  for (int r = 0; r < 12; r++) read_one(f0, r, wd_lds, 0);

  int st = 0;  // stage of the current step
  const bool vec_ok = (p.ldc & 7) == 0 && ((uintptr_t)p.c & 15) == 0;
  for (int lin = first; lin < tiles; lin += G) {
    int row0, n0;
    tile_origin(lin, row0, n0);
    for (int kt = 0; kt < nk; kt++) {
      const uint8_t* cur_sb = wd_lds + st * WD_STAGE;
      const uint8_t* oth_sb = wd_lds + (st ^ 1) * WD_STAGE;
      half_step(f0, f1, cur_sb, 1, std::false_type{}, 0);
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __syncthreads();  // the next step has landed everywhere; this stage has been read by everyone
      __builtin_amdgcn_sched_barrier(0);
      half_step(f1, f0, oth_sb, 0, std::true_type{}, st);
      advance_loads();
      st ^= 1;
    }

    // ---- epilogue: lane holds C[row0 + 128 wm + 16 i + r16][n0 + 64 wn + 16 g + 4 j + c]
    const int nb = n0 + 64 * wn + 16 * g;
    float bv[16];
    if (p.bias) {
#pragma unroll
      for (int e = 0; e < 16; e++) bv[e] = bf16_to_f32(p.bias[min(nb + e, N - 1)]);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int m = row0 + 128 * wm + 16 * i + r16;
      bf16_t o[16];
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          float v = acc[i][j][c];
          if (p.bias) v += bv[4 * j + c];
          o[4 * j + c] = f32_to_bf16(v);
          acc[i][j][c] = 0.f;
        }
      if (m >= M) continue;
      bf16_t* cp = p.c + (int64_t)m * p.ldc + nb;
      if (vec_ok && nb + 15 < N) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
          uint4 pk;
          pk.x = (uint32_t)o[8 * h + 0] | ((uint32_t)o[8 * h + 1] << 16);
          pk.y = (uint32_t)o[8 * h + 2] | ((uint32_t)o[8 * h + 3] << 16);
          pk.z = (uint32_t)o[8 * h + 4] | ((uint32_t)o[8 * h + 5] << 16);
          pk.w = (uint32_t)o[8 * h + 6] | ((uint32_t)o[8 * h + 7] << 16);
          *(uint4*)(cp + 8 * h) = pk;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 16; e++)
          if (nb + e < N) cp[e] = o[e];
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // loads past the last step still target our LDS
}

// Launches the wide kernel. Returns false (nothing launched) when the shape does not qualify.
static inline bool gemm_wide_launch(const GemmParams& p, hipStream_t stream) {
  if (p.K % WD_BK != 0 || p.M <= 0 || p.N <= 0) return false;
  const int64_t lim = (int64_t)1 << 32;
  if (((int64_t)p.M * p.ldx + p.K) * 2 >= lim || ((int64_t)p.N * p.ldw + p.K) * 2 >= lim) return false;
  static bool attr_set = false;  // per process; the attribute is a property of the loaded function
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)gemm_wide_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            WD_LDS) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    attr_set = true;
  }
  const int64_t tm = ((int64_t)p.M + WD_BM - 1) / WD_BM, tn = ((int64_t)p.N + WD_BN - 1) / WD_BN;
  const int64_t tiles = tm * tn;
  if (tiles > (1 << 30)) return false;
  const unsigned grid = (unsigned)(tiles >= 256 ? 256 : (tiles + 7) / 8 * 8);
  gemm_wide_kernel<<<grid, 512, WD_LDS, stream>>>(p, (int)tm, (int)tn);
  return true;
}

}  // namespace vx
