// Wide-tile bf16 "NT" GEMM for many rows (prefill): C[m, n] = r16(sum_k X[m, k] W[n, k] (+ bias[n])).
//
// One workgroup = 8 wavefronts (two per SIMD) computes a 256 (activation rows) x 256 (weight rows)
// tile, 64 k-elements per step. Both operand tiles go HBM/L2 -> LDS directly
// (global_load_lds_dwordx4: a wavefront writes 1 KB = 8 tile rows of 128 bytes per instruction, no
// staging registers, no ds_write), two stages of 64 KB each, one barrier per step. The 16-byte
// pieces of a tile row are stored XOR-swizzled by (row >> 1) & 7 - the lane that fills slot s of row
// R fetches logical piece s ^ swz(R) - so the 16 rows x 16 bytes of one MFMA fragment read hit 64
// distinct banks although the rows are unpadded.
// Wavefront (wm, wn) of the 2 x 4 arrangement owns activation rows [128 wm, +128) and weight rows
// [64 wn, +64): 8 x 4 MFMA tiles, 12 fragment reads per 32 MFMAs.
// Arithmetic per output element is the same as in the other GEMM kernels (A = weight fragment,
// B = activation fragment, K ascending in 32-chunks), so results are bit-identical to theirs.
// Requirements (checked by the host): K % 64 == 0, 16-byte aligned rows. Rows past M / N are clamped
// on load (a C row only depends on its own X row, a column on its own W row) and masked on store.
//
// Workgroup -> tile mapping: consecutive workgroup ids go to different XCDs (id % 8), each with its
// own L2, so the ids are regrouped such that one XCD works through a contiguous run of tiles, and the
// run is ordered in panels of 4 row tiles x all column tiles: the ~32 tiles in flight on an XCD then
// share 4 activation panels and 8 weight panels.
#pragma once
#include "gemm_core.h"

#ifndef WD_EXP
#define WD_EXP 0
#endif
namespace vx {

constexpr int WD_BM = 256, WD_BN = 256, WD_BK = 64;
constexpr int WD_XBYTES = WD_BM * WD_BK * 2;             // 32 KB
constexpr int WD_STAGE = (WD_BM + WD_BN) * WD_BK * 2;    // 64 KB
constexpr int WD_LDS = 2 * WD_STAGE;                     // 128 KB
constexpr int WD_GROUP_M = 4;

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

__global__ __launch_bounds__(512) void gemm_wide_kernel(GemmParams p, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t wd_lds[];

  // ---- tile of this workgroup
  const int per_xcd = gridDim.x >> 3;
  const int lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (lin >= tiles_m * tiles_n) return;
  const int span = WD_GROUP_M * tiles_n;
  const int grp = lin / span;
  const int gm0 = grp * WD_GROUP_M;
  const int gsz = min(WD_GROUP_M, tiles_m - gm0);
  const int rem = lin - grp * span;
  const int row0 = (gm0 + rem % gsz) * WD_BM;
  const int n0 = (rem / gsz) * WD_BN;

  const int M = p.M, N = p.N, K = p.K;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int wm = wave >> 2, wn = wave & 3;

  // ---- loads: instruction j of this wavefront fills tile rows [8 (wave + 8 j), +8) of X and of W
  const int lrow = lane >> 3, lslot = lane & 7;
  const bf16_t* xg[4];
  const bf16_t* wg[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int R = 8 * (wave + 8 * j) + lrow;
    const int c = lslot ^ ((R >> 1) & 7);
    xg[j] = p.x + (int64_t)min(row0 + R, M - 1) * p.ldx + c * 8;
    wg[j] = p.w + (int64_t)min(n0 + R, N - 1) * p.ldw + c * 8;
  }
  // The loads are written as asm so that the compiler does not track them: told that they write LDS,
  // it would wait for them (vmcnt(0)) before the first fragment read of the step they are issued in.
  // The wait that matters is the explicit one before the barrier of the step that consumes them.
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)wd_lds + wave * 1024;
  auto issue = [&](int stage, int k0) {
    const uint32_t sb = lds0 + stage * WD_STAGE;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                   :: "s"(sb + j * 8192), "v"(xg[j] + k0) : "memory", "m0");
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                   :: "s"(sb + WD_XBYTES + j * 8192), "v"(wg[j] + k0) : "memory", "m0");
    }
  };

  f32x4 acc[8][4];  // [activation tile i][weight tile j]
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // fragment read offsets: row (tile base + r16), logical piece 4 ks + g, slot = piece ^ (r16 >> 1)
  const int slot0 = (g ^ (r16 >> 1)) * 16;
  const int xoff = (128 * wm + r16) * 128;
  const int woff = WD_XBYTES + (64 * wn + r16) * 128;

  // Fragments of one 32-wide k-step: 4 weight (A) and 8 activation (B) operands.
  struct Frag { uint4 w[4], x[8]; };
  auto read_frag = [&](Frag& f, int stage, int ks) {
    const uint8_t* sb = wd_lds + stage * WD_STAGE + (slot0 ^ (64 * ks));
#pragma unroll
    for (int j = 0; j < 4; j++) f.w[j] = *(const uint4*)(sb + woff + j * 2048);
#pragma unroll
    for (int i = 0; i < 8; i++) f.x[i] = *(const uint4*)(sb + xoff + i * 2048);
  };
  auto mma = [&](const Frag& f) {
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) acc[i][j] = mfma16(f.w[j], f.x[i], acc[i][j]);
  };

  // Software pipeline: fragment reads run one MFMA block ahead, global loads two steps ahead. The
  // barrier of step kt sits between its two MFMA blocks: by then every wavefront has read both
  // halves of stage kt (so the stage can be refilled with step kt+2) and step kt+1 has landed.
  const int nk = K / WD_BK;
  Frag f0, f1;
  issue(0, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (nk > 1) issue(1, WD_BK);
  read_frag(f0, 0, 0);
  for (int kt = 0; kt < nk; kt++) {
#if WD_EXP != 1
    read_frag(f1, kt & 1, 1);
#endif
    mma(f0);
    __builtin_amdgcn_sched_barrier(0);  // keep the MFMA block in front of the wait
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
#if WD_EXP != 2
    if (kt + 2 < nk) issue(kt & 1, (kt + 2) * WD_BK);
#endif
#if WD_EXP != 1
    if (kt + 1 < nk) read_frag(f0, (kt + 1) & 1, 0);
    mma(f1);
#else
    mma(f0);
#endif
  }

  // ---- epilogue: lane holds C[row0 + 128 wm + 16 i + r16][n0 + 64 wn + 16 j + 4 g + c]
  const bool vec_ok = (p.ldc & 3) == 0;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int m = row0 + 128 * wm + 16 * i + r16;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int nc = n0 + 64 * wn + 16 * j + 4 * g;
      bf16_t* cp = p.c + (int64_t)m * p.ldc + nc;
      bf16_t o[4];
#pragma unroll
      for (int c = 0; c < 4; c++) {
        float v = acc[i][j][c];
        if (p.bias && nc + c < N) v += bf16_to_f32(p.bias[nc + c]);
        o[c] = f32_to_bf16(v);
      }
      if (nc + 3 < N && vec_ok) {
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

// Launches the wide kernel. Returns false (nothing launched) when the shape does not qualify.
static inline bool gemm_wide_launch(const GemmParams& p, hipStream_t stream) {
  if (p.K % WD_BK != 0 || p.M <= 0 || p.N <= 0) return false;
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
  const unsigned grid = (unsigned)((tiles + 7) / 8 * 8);
  gemm_wide_kernel<<<grid, 512, WD_LDS, stream>>>(p, (int)tm, (int)tn);
  return true;
}

}  // namespace vx
