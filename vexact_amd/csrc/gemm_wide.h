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
constexpr int WD_GROUP_M = 4;

typedef __attribute__((address_space(3))) void* lptr_t;
typedef uint32_t u32x4_nt __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int wd_swz_x(int R) { return (R >> 1) & 7; }
__device__ __forceinline__ int wd_swz_w(int R) { return (((R >> 4) & 3) << 1) | ((R >> 1) & 1); }

// One tile of the walk: rows [row0, row0 + rows) of C, output columns from n0, weights at wbase.
struct WideTile {
  int row0, rows, n0;
  int64_t wbase;
  bool ok;
};

// GROUPED (MoE expert GEMMs at prefill sizes): row tiles come from the tile table of the routing
// kernel (group, first row, row count; built for 256-row tiles, compact, -1 after the last used
// entry), activation rows may be gathered through row_src, and tiles are numbered row-tile major, so
// the workgroups of an XCD share one expert's weights and a few activation panels. tiles_m is then
// the length of the table.
// EPI_SWIGLU: the 256 weight rows of a tile are 128 gate rows and the 128 up rows of the same
// output columns, interleaved so that wavefront wn holds gate columns [32 wn, +32) in its weight
// fragments 0, 1 and the matching up columns in fragments 2, 3: LDS row 64 wn + 16 a + 4 j + b is
// column 32 wn + 8 a + 4 (j & 1) + b of gate (j < 2) or up (j >= 2). A tile then yields 128 output
// columns and a lane 8 consecutive ones per activation row.
// XI = 16-row activation tiles per wavefront: 8 (256-row tiles, the normal form) or 4 (128-row tiles: the same
// weight panel and barriers for half the rows, for a last round of tiles that would leave half the chip idle).
// PACKED: the weights are in fragment order (pack_weights_kernel; p.ldw = 32-wide k-chunks stored per 16-row
// block; a step advances two chunks = 1024 elements). There 16-byte piece pc (8 k-elements) of the 16 rows of a
// block is contiguous, so the weight tile lives in LDS piece-major and in fragment order, [pc][position] with
// position 64 wn + 16 j + rho for MFMA row rho of wavefront wn's weight fragment j: a load instruction fills
// the 64 positions of one (pc, wn) from 4 blocks x 256 contiguous bytes (whole lines, 4 consecutive lanes on 64
// contiguous bytes, as with row-major weights), and a fragment read takes 256 contiguous LDS bytes per 16 lanes
// (no swizzle needed). With the SwiGLU epilogue an instruction mixes gate rows (j < 2) and up rows, so the up
// image's distance from the gate image is part of the lane offset (host check: w2 behind w, within 4 GiB).
template <int EPI, bool GROUPED, int XI = 8, bool PACKED = false>
__global__ __launch_bounds__(512) void gemm_wide_kernel(GemmParams p, int tiles_m, int tiles_n) {
  static_assert(!PACKED || GROUPED, "fragment-order weights exist for the grouped form only");
  extern __shared__ __attribute__((aligned(1024))) uint8_t wd_lds[];
  constexpr int NOUT = (EPI == EPI_SWIGLU) ? 128 : 256;  // output columns per tile
  constexpr int BM = 32 * XI;                             // activation rows per tile
  constexpr int NXQ = BM / 64;                            // activation load instructions per wavefront and step
  constexpr int NLQ = NXQ + 4;                            // all load instructions per wavefront and step
  constexpr int XBYTES = BM * WD_BK * 2;
  constexpr int STAGE = XBYTES + WD_BN * WD_BK * 2;
  static_assert(XI == 8 || XI == 4, "wavefront tile heights");

  const int N = p.N, K = p.K;
  const int tiles = tiles_m * tiles_n;
  const int G = gridDim.x;  // multiple of 8
  const int first = (blockIdx.x & 7) * (G >> 3) + (blockIdx.x >> 3);

  auto tile_at = [&](int lin) {
    WideTile t;
    if constexpr (GROUPED) {
      const int mt = lin / tiles_n;
      const int grp = p.tile_group[mt];
      t.ok = grp >= 0;
      t.row0 = p.tile_row0[mt];
      t.rows = p.tile_rows[mt];
      t.n0 = (lin - mt * tiles_n) * NOUT;
      t.wbase = (int64_t)(t.ok ? grp : 0) * p.w_gstride;
    } else {
      const int span = WD_GROUP_M * tiles_n;
      const int grp = lin / span;
      const int gm0 = grp * WD_GROUP_M;
      const int gsz = min(WD_GROUP_M, tiles_m - gm0);
      const int rem = lin - grp * span;
      t.row0 = (gm0 + rem % gsz) * BM;
      t.rows = min(BM, p.M - t.row0);
      t.n0 = (rem / gsz) * NOUT;
      t.wbase = 0;
      t.ok = true;
    }
    return t;
  };
  if (first >= tiles || !tile_at(first).ok) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int wm = wave >> 2, wn = wave & 3;

  // ---- load stream: instruction q of a step fills tile rows [8 (wave + 8 q), +8) of X (q < NXQ)
  // or rows [8 (wave + 8 (q - NXQ)), +8) of W. Byte offsets from the operand base fit 32 bits (host check).
  const int lrow = lane >> 3, lslot = lane & 7;
  uint32_t ld_off[NLQ];
  int64_t ld_wbase = 0;
  auto set_load_tile = [&](const WideTile& t) {
    // wave-uniform by construction; said explicitly so that the loads' scalar base stays in scalar registers
    // whatever the surrounding code makes the compiler choose
    ld_wbase = (int64_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)((uint64_t)t.wbase >> 32)) << 32) |
                         (uint32_t)__builtin_amdgcn_readfirstlane((int)t.wbase));
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int R = 8 * (wave + 8 * j) + lrow;
      if (j < NXQ) {
        const int rr = t.row0 + min(R, t.rows - 1);  // rows past the tile re-read its last row (not stored)
        const int64_t sr = (GROUPED && p.row_src) ? (int64_t)p.row_src[rr] : (int64_t)rr;
        ld_off[j] = (uint32_t)((sr * p.ldx + (lslot ^ wd_swz_x(R)) * 8) * 2);
      }
      // tile row (in the numbering of the row-major LDS layout) and 16-byte piece that this lane fetches
      int Rw, pc;
      if constexpr (PACKED) {
        const int qq = wave + 8 * j;  // instruction (pc, wn) = (qq / 4, qq % 4) fills positions 64 wn + lane
        pc = qq >> 2;
        Rw = 64 * (qq & 3) + 16 * ((lane & 15) >> 2) + 4 * (lane >> 4) + (lane & 3);
      } else {
        Rw = R;
        pc = lslot ^ wd_swz_w(R);
      }
      int col;
      if constexpr (EPI == EPI_SWIGLU) col = t.n0 + 32 * (Rw >> 6) + 8 * ((Rw >> 4) & 3) + 4 * ((Rw >> 2) & 1) + (Rw & 3);
      else col = t.n0 + Rw;
      if constexpr (PACKED) {
        const int cc = min(col, N - 1);
        int64_t off = (((int64_t)(cc >> 4) * p.ldw + (pc >> 2)) * 512 + ((cc & 15) + 16 * (pc & 3)) * 8) * 2;
        if (EPI == EPI_SWIGLU && ((Rw >> 3) & 1)) off += (int64_t)((const uint8_t*)p.w2 - (const uint8_t*)p.w);
        ld_off[NXQ + j] = (uint32_t)off;
      } else {
        ld_off[NXQ + j] = (uint32_t)(((int64_t)min(col, N - 1) * p.ldw + pc * 8) * 2);
      }
    }
  };
  int ld_lin = first, ld_k = 0;
  set_load_tile(tile_at(first));
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)wd_lds + wave * 1024;
  // EPI_SWIGLU: weight rows 8 q .. 8 q + 7 of load instruction q = wave + 8 j have bit 3 of the row
  // index equal to the parity of the wavefront, which says gate or up
  const bf16_t* wsrc = (EPI == EPI_SWIGLU && !PACKED && (wave & 1)) ? p.w2 : p.w;
  // The loads are written as asm so that the compiler does not track them: told that they write LDS,
  // it would wait for them (vmcnt(0)) before the first fragment read after they are issued. The
  // wait that matters is the explicit one before the barrier that precedes their first use.
  auto issue_one = [&](int q, int stage) {
    const uint32_t dst = lds0 + stage * STAGE + (q < NXQ ? q * 8192 : XBYTES + (q - NXQ) * 8192);
    const bf16_t* base = q < NXQ ? p.x + ld_k : wsrc + ld_wbase + (PACKED ? 16 * ld_k : ld_k);
    lds_load16_sv(dst, ld_off[q], base);
  };
  auto advance_loads = [&]() {  // next step of the stream; past the last tile it re-reads (unused)
    ld_k += WD_BK;
    if (ld_k >= K) {
      ld_k = 0;
      const int nl = ld_lin + G;
      if (nl < tiles) {
        const WideTile t = tile_at(nl);
        if (t.ok) {
          ld_lin = nl;
          set_load_tile(t);
        }
      }
    }
  };

  f32x4 acc[XI][4];  // [activation tile i][weight tile j]
#pragma unroll
  for (int i = 0; i < XI; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- fragment reads, k-half 0; k-half 1 is the same address with bit 6 flipped (slot ^ 4).
  // Activation rows 16 XI wm + 16 i + r16: swizzle term r16 >> 1. Weight rows
  // 64 wn + 16 (r16 / 4) + 4 j + r16 % 4: swizzle term 2 (r16 / 4) + (r16 % 4) / 2.
  const int xoff = (16 * XI * wm + r16) * 128 + ((g ^ (r16 >> 1)) * 16);
  const int woff = PACKED ? XBYTES + g * 4096 + (64 * wn + r16) * 16
                          : XBYTES + (64 * wn + 16 * (r16 >> 2) + (r16 & 3)) * 128 +
                                ((g ^ (((r16 >> 2) << 1) | ((r16 >> 1) & 1))) * 16);
  struct Frag { uint4 w[4], x[XI]; };
  // read number r (0 .. 3 + XI) of a fragment set: the 4 weight operands first, then the XI activation ones
  auto read_one = [&](Frag& f, int r, const uint8_t* sb, int ks) {
    if (r < 4) f.w[r] = PACKED ? *(const uint4*)(sb + woff + ks * 16384 + r * 256) : *(const uint4*)(sb + (woff ^ (64 * ks)) + r * 512);
    else f.x[r - 4] = *(const uint4*)(sb + (xoff ^ (64 * ks)) + (r - 4) * 2048);
  };
  // 4 XI MFMAs on `cur`, interleaved with the 4 + XI reads of `nxt` and (LOADS) the global loads of a step
  auto half_step = [&](const Frag& cur, Frag& nxt, const uint8_t* nxt_sb, int nxt_ks, auto LOADS,
                       int ld_stage) {
#pragma unroll
    for (int i = 0; i < XI; i++) {
#pragma unroll
      for (int j = 0; j < 4; j++) acc[i][j] = mfma16(cur.w[j], cur.x[i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (decltype(LOADS)::value) {
        if (2 * i < NLQ) {
          issue_one(2 * i, ld_stage);
          issue_one(2 * i + 1, ld_stage);
        }
      }
      if (i < 4) {  // two reads beside each of the first four MFMA groups, one beside the others (XI = 8)
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
  for (int q = 0; q < NLQ; q++) issue_one(q, 0);
  advance_loads();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
#pragma unroll
  for (int q = 0; q < NLQ; q++) issue_one(q, 1);
  advance_loads();
#pragma unroll
  for (int r = 0; r < 4 + XI; r++) read_one(f0, r, wd_lds, 0);

  int st = 0;  // stage of the current step
  const bool vec_ok = (p.ldc & 7) == 0 && ((uintptr_t)p.c & 15) == 0;
  for (int lin = first; lin < tiles; lin += G) {
    const WideTile t = tile_at(lin);
    if (!t.ok) break;
    for (int kt = 0; kt < nk; kt++) {
      const uint8_t* cur_sb = wd_lds + st * STAGE;
      const uint8_t* oth_sb = wd_lds + (st ^ 1) * STAGE;
      half_step(f0, f1, cur_sb, 1, std::false_type{}, 0);
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __syncthreads();  // the next step has landed everywhere; this stage has been read by everyone
      __builtin_amdgcn_sched_barrier(0);
      half_step(f1, f0, oth_sb, 0, std::true_type{}, st);
      advance_loads();
      st ^= 1;
    }

    if constexpr (EPI == EPI_SWIGLU) {
      // lane holds gate (fragments 0, 1) and up (2, 3) of columns n0 + 32 wn + 8 g + 4 j + c
      const int nb = t.n0 + 32 * wn + 8 * g;
#pragma unroll
      for (int i = 0; i < XI; i++) {
        const int m = 16 * XI * wm + 16 * i + r16;
        float wr = 0.f;
        if (m < t.rows) {
          const int64_t orow = t.row0 + m;
          wr = p.row_scale ? bf16_to_f32(p.row_scale[p.row_scale_idx ? p.row_scale_idx[orow] : (int)orow]) : 1.0f;
        }
        bf16_t o[8];
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
          for (int c = 0; c < 4; c++) {
            o[4 * j + c] = swiglu_bf16(acc[i][j][c], acc[i][j + 2][c], wr);
            acc[i][j][c] = 0.f;
            acc[i][j + 2][c] = 0.f;
          }
        if (m >= t.rows) continue;
        bf16_t* cp = p.c + (int64_t)(t.row0 + m) * p.ldc + nb;
        if (vec_ok && nb + 7 < N) {
          uint4 pk;
          pk.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
          pk.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
          pk.z = (uint32_t)o[4] | ((uint32_t)o[5] << 16);
          pk.w = (uint32_t)o[6] | ((uint32_t)o[7] << 16);
          __builtin_nontemporal_store(__builtin_bit_cast(u32x4_nt, pk), (u32x4_nt*)cp);
        } else {
#pragma unroll
          for (int e = 0; e < 8; e++)
            if (nb + e < N) cp[e] = o[e];
        }
      }
    } else {
      // lane holds C[row0 + 16 XI wm + 16 i + r16][n0 + 64 wn + 16 g + 4 j + c]
      const int nb = t.n0 + 64 * wn + 16 * g;
      float bv[16];
      if (p.bias) {
#pragma unroll
        for (int e = 0; e < 16; e++) bv[e] = bf16_to_f32(p.bias[min(nb + e, N - 1)]);
      }
#pragma unroll
      for (int i = 0; i < XI; i++) {
        const int m = 16 * XI * wm + 16 * i + r16;
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
        if (m >= t.rows) continue;
        bf16_t* cp = p.c + (int64_t)(t.row0 + m) * p.ldc + nb;
        if (vec_ok && nb + 15 < N) {
#pragma unroll
          for (int h = 0; h < 2; h++) {
            uint4 pk;
            pk.x = (uint32_t)o[8 * h + 0] | ((uint32_t)o[8 * h + 1] << 16);
            pk.y = (uint32_t)o[8 * h + 2] | ((uint32_t)o[8 * h + 3] << 16);
            pk.z = (uint32_t)o[8 * h + 4] | ((uint32_t)o[8 * h + 5] << 16);
            pk.w = (uint32_t)o[8 * h + 6] | ((uint32_t)o[8 * h + 7] << 16);
            __builtin_nontemporal_store(__builtin_bit_cast(u32x4_nt, pk), (u32x4_nt*)(cp + 8 * h));
          }
        } else {
#pragma unroll
          for (int e = 0; e < 16; e++)
            if (nb + e < N) cp[e] = o[e];
        }
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // loads past the last step still target our LDS
}

// Launch helper shared by the dense and the grouped entry points. x_rows = rows addressable in x
// (bounds the 32-bit load offsets). Returns false (nothing launched) when the shape does not qualify.
template <int EPI, bool GROUPED, int XI = 8, bool PACKED = false>
static inline bool gemm_wide_launch_t(const GemmParams& p, int64_t tiles_m, int64_t x_rows, hipStream_t stream) {
  constexpr int NOUT = (EPI == EPI_SWIGLU) ? 128 : 256;
  constexpr int LDS = 2 * (32 * XI + WD_BN) * WD_BK * 2;  // two stages of an activation and a weight tile
  if (p.K % WD_BK != 0 || p.N <= 0 || tiles_m <= 0 || x_rows <= 0) return false;
  const int64_t lim = (int64_t)1 << 32;
  // bytes of one group's weights that a load offset must reach (PACKED: 16-row blocks of p.ldw 1 KB chunks)
  int64_t wspan = PACKED ? (((int64_t)p.N + 15) / 16) * p.ldw * 1024 : ((int64_t)p.N * p.ldw + p.K) * 2;
  if (PACKED && EPI == EPI_SWIGLU) {  // up rows are addressed from the gate image
    const int64_t delta = (const uint8_t*)p.w2 - (const uint8_t*)p.w;
    if (delta < 0) return false;
    wspan += delta;
  }
  if ((x_rows * p.ldx + p.K) * 2 >= lim || wspan >= lim) return false;
  const int64_t tn = ((int64_t)p.N + NOUT - 1) / NOUT;
  const int64_t tiles = tiles_m * tn;
  if (tiles > (1 << 30)) return false;
  static DeviceOnce once;  // per instantiation
  const int dev = once.slot();
  if (once.need(dev)) {
    if (hipFuncSetAttribute((const void*)gemm_wide_kernel<EPI, GROUPED, XI, PACKED>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    once.mark(dev);
  }
  const unsigned grid = (unsigned)(tiles >= 256 ? 256 : (tiles + 7) / 8 * 8);
  gemm_wide_kernel<EPI, GROUPED, XI, PACKED><<<grid, 512, LDS, stream>>>(p, (int)tiles_m, (int)tn);
  return true;
}

// Columns [0, n1) of a dense product go to 256-row tiles and [n1, N) to 128-row tiles when the 256 x 256 tiles'
// last round would fill at most half of the 256 workgroups (640 tiles: two rounds of 256-row tiles over the
// first 512, then one round of 256 half-height tiles instead of a third round on 128 workgroups). A half-height
// tile pays the whole weight panel and every barrier for half the rows (measured ~0.7 of a full tile), so only
// such a last round gains: the q/k/v projection of an 8192-token chunk 154 -> 147 us. With few row tiles the
// kernel streams weights from HBM and a half-height tile costs what a full one does (lm_head at 256 rows:
// 206 us either way), so those shapes are left alone. Returns N when there is nothing to split.
static inline int64_t gemm_wide_split_col(int64_t M, int64_t N, int nout) {
  const int64_t tm = (M + WD_BM - 1) / WD_BM, tn = (N + nout - 1) / nout;
  const int64_t rem = (tm * tn) % 256;
  if (tm < 4 || tm * tn < 256 || rem == 0 || rem > 128) return N;
  // the fewest trailing column tiles whose removal leaves whole rounds
  for (int64_t cut = 1; cut < tn && tm * cut <= 128; cut++)
    if ((tm * (tn - cut)) % 256 == 0) return (tn - cut) * nout;
  return N;
}

// dense: C[M, N] = X W^T (+ bias)
static inline bool gemm_wide_launch(const GemmParams& p, hipStream_t stream) {
  if (p.M <= 0) return false;
  const int64_t n1 = gemm_wide_split_col(p.M, p.N, WD_BN);
  if (n1 == p.N) return gemm_wide_launch_t<EPI_PLAIN, false>(p, ((int64_t)p.M + WD_BM - 1) / WD_BM, p.M, stream);
  GemmParams a = p, b = p;
  a.N = (int)n1;
  b.N = p.N - (int)n1;
  b.w = p.w + n1 * p.ldw;
  b.c = p.c + n1;
  if (p.bias) b.bias = p.bias + n1;
  if (!gemm_wide_launch_t<EPI_PLAIN, false>(a, ((int64_t)p.M + WD_BM - 1) / WD_BM, p.M, stream)) return false;
  return gemm_wide_launch_t<EPI_PLAIN, false, 4>(b, ((int64_t)p.M + 127) / 128, p.M, stream);
}

// dense with the SwiGLU epilogue: C[M, N] = swiglu(X Wg^T, X Wu^T)
static inline bool gemm_wide_swiglu_launch(const GemmParams& p, hipStream_t stream) {
  if (p.M <= 0) return false;
  return gemm_wide_launch_t<EPI_SWIGLU, false>(p, ((int64_t)p.M + WD_BM - 1) / WD_BM, p.M, stream);
}

// grouped, over a 256-row tile table of max_m_tiles entries
static inline bool gemm_wide_grouped_launch(const GemmParams& p, int epi, int64_t max_m_tiles, int64_t x_rows,
                                            hipStream_t stream) {
  if (epi == EPI_SWIGLU) return gemm_wide_launch_t<EPI_SWIGLU, true>(p, max_m_tiles, x_rows, stream);
  return gemm_wide_launch_t<EPI_PLAIN, true>(p, max_m_tiles, x_rows, stream);
}
// the same on fragment-order weights (p.ldw = k-chunks per 16-row block)
static inline bool gemm_wide_grouped_packed_launch(const GemmParams& p, int epi, int64_t max_m_tiles, int64_t x_rows,
                                                   hipStream_t stream) {
  if (epi == EPI_SWIGLU) return gemm_wide_launch_t<EPI_SWIGLU, true, 8, true>(p, max_m_tiles, x_rows, stream);
  return gemm_wide_launch_t<EPI_PLAIN, true, 8, true>(p, max_m_tiles, x_rows, stream);
}

// ---------------------------------------------------------------------------------------
// Ring kernel for a few hundred rows (decode-sized batches against dense weights), where one
// wavefront's chain of dependent HBM round trips, not bandwidth, bounds the streaming kernel.
// 4 wavefronts (2 x 2) compute a (32 XF) x (32 WF) tile; both operands go directly to LDS
// (same swizzled 128-byte rows as the wide kernel) into a ring of S stages of 64 k-elements, so
// S - 1 steps of loads are in flight per workgroup whatever the compute does. One barrier per step;
// the loads of step s + S - 1 refill the stage that was read in step s - 1. Past the last step the
// ring keeps loading (valid addresses, unread stages) so that the outstanding-load count the
// waits rely on stays constant.
// ---------------------------------------------------------------------------------------
template <int XF, int WF, int S, int KSUB>
__global__ __launch_bounds__(256) void gemm_ring_kernel(GemmParams p) {
  constexpr int BM = 32 * XF, BN = 32 * WF, BK = 64 * KSUB;
  constexpr int XB = BM * 128, SUB = (BM + BN) * 128, STAGE = KSUB * SUB;
  constexpr int NSUB = (BM + BN) / 8;  // wavefront-wide load instructions per 64-wide sub-tile
  constexpr int NLD = KSUB * NSUB;     // per step
  constexpr int LPW = NLD / 4;         // per wavefront
  static_assert(NLD % 4 == 0, "loads must split evenly over the 4 wavefronts");
  static_assert((S - 2) * LPW <= 63, "vmcnt field");
  extern __shared__ __attribute__((aligned(1024))) uint8_t rg_lds[];

  const int M = p.M, N = p.N, K = p.K;
  const int row0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;

  // load instruction q = wave + 4 t: sub-tile q / NSUB, rows [8 (q % NSUB), +8) of X (first BM / 8) or W
  const int lrow = lane >> 3, lslot = lane & 7;
  uint32_t ld_off[LPW];
#pragma unroll
  for (int t = 0; t < LPW; t++) {
    const int q = (wave + 4 * t) % NSUB;
    if (q < BM / 8) {
      const int R = 8 * q + lrow;
      ld_off[t] = (uint32_t)(((int64_t)min(row0 + R, M - 1) * p.ldx + (lslot ^ wd_swz_x(R)) * 8) * 2);
    } else {
      const int R = 8 * (q - BM / 8) + lrow;
      const int sw = (((R / (4 * WF)) & 3) << 1) | ((R >> 1) & 1);
      ld_off[t] = (uint32_t)(((int64_t)min(n0 + R, N - 1) * p.ldw + (lslot ^ sw) * 8) * 2);
    }
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)rg_lds;
  const int nk = K / BK;  // K % BK == 0 (host check)
  auto issue = [&](int step) {  // loads of `step` (wrapped past the end) into stage step % S
    const int st = step < nk ? step : step % nk;
    const uint32_t sb = lds0 + (step % S) * STAGE;
#pragma unroll
    for (int t = 0; t < LPW; t++) {
      const int qq = wave + 4 * t;  // wave-uniform
      const int u = qq / NSUB, q = qq % NSUB;
      const bool isx = q < BM / 8;
      const uint32_t dst = sb + u * SUB + (isx ? q * 1024 : XB + (q - BM / 8) * 1024);
      const bf16_t* base = (isx ? p.x : p.w) + (st * KSUB + u) * 64;
      lds_load16_sv(dst, ld_off[t], base);
    }
  };

  f32x4 acc[XF][WF];
#pragma unroll
  for (int i = 0; i < XF; i++)
#pragma unroll
    for (int j = 0; j < WF; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // fragment addresses (k-half 0; k-half 1 flips bit 6). Weight fragment j, MFMA row rho is weight
  // row 4 WF (rho / 4) + 4 j + rho % 4 of the wavefront's 16 WF: a lane's outputs are contiguous in n.
  const int xoff = (16 * XF * wm + r16) * 128 + ((g ^ (r16 >> 1)) * 16);
  const int woff = XB + (16 * WF * wn + 4 * WF * (r16 >> 2) + (r16 & 3)) * 128 +
                   ((g ^ (((r16 >> 2) << 1) | ((r16 >> 1) & 1))) * 16);

#pragma unroll
  for (int t = 0; t < S - 1; t++) issue(t);
  for (int s = 0; s < nk; s++) {
    // in-order completion: at most the S - 2 youngest steps may still be in flight
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"((S - 2) * LPW) : "memory");
    __syncthreads();  // step s is in LDS for everyone; everyone is done reading step s - 1
    issue(s + S - 1);
    const uint8_t* sb = rg_lds + (s % S) * STAGE;
    // all fragment reads of the step first, then its MFMAs: one LDS round trip per step
    uint4 wf[2 * KSUB][WF], xf[2 * KSUB][XF];
#pragma unroll
    for (int kk = 0; kk < 2 * KSUB; kk++) {
      const uint8_t* sk = sb + (kk >> 1) * SUB;
#pragma unroll
      for (int j = 0; j < WF; j++) wf[kk][j] = *(const uint4*)(sk + (woff ^ (64 * (kk & 1))) + j * 512);
#pragma unroll
      for (int i = 0; i < XF; i++) xf[kk][i] = *(const uint4*)(sk + (xoff ^ (64 * (kk & 1))) + i * 2048);
    }
#pragma unroll
    for (int kk = 0; kk < 2 * KSUB; kk++)
#pragma unroll
      for (int i = 0; i < XF; i++)
#pragma unroll
        for (int j = 0; j < WF; j++) acc[i][j] = mfma16(wf[kk][j], xf[kk][i], acc[i][j]);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the ring's trailing loads still target our LDS

  // epilogue: lane holds C[row0 + 16 XF wm + 16 i + r16][n0 + 16 WF wn + 4 WF g + 4 j + c]
  const int nb = n0 + 16 * WF * wn + 4 * WF * g;
  const bool vec_ok = (p.ldc & 7) == 0 && ((uintptr_t)p.c & 15) == 0;
#pragma unroll
  for (int i = 0; i < XF; i++) {
    const int m = row0 + 16 * XF * wm + 16 * i + r16;
    if (m >= M) continue;
    bf16_t o[4 * WF];
#pragma unroll
    for (int j = 0; j < WF; j++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        float v = acc[i][j][c];
        if (p.bias) v += bf16_to_f32(p.bias[min(nb + 4 * j + c, N - 1)]);
        o[4 * j + c] = f32_to_bf16(v);
      }
    bf16_t* cp = p.c + (int64_t)m * p.ldc + nb;
    if (vec_ok && WF % 2 == 0 && nb + 4 * WF - 1 < N) {
#pragma unroll
      for (int h = 0; h < WF / 2; h++) {
        uint4 pk;
        pk.x = (uint32_t)o[8 * h + 0] | ((uint32_t)o[8 * h + 1] << 16);
        pk.y = (uint32_t)o[8 * h + 2] | ((uint32_t)o[8 * h + 3] << 16);
        pk.z = (uint32_t)o[8 * h + 4] | ((uint32_t)o[8 * h + 5] << 16);
        pk.w = (uint32_t)o[8 * h + 6] | ((uint32_t)o[8 * h + 7] << 16);
        *(uint4*)(cp + 8 * h) = pk;
      }
    } else if (WF == 1 && (p.ldc & 3) == 0 && ((uintptr_t)p.c & 7) == 0 && nb + 3 < N) {
      uint2 pk;
      pk.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
      pk.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
      *(uint2*)cp = pk;
    } else {
#pragma unroll
      for (int e = 0; e < 4 * WF; e++)
        if (nb + e < N) cp[e] = o[e];
    }
  }
}

template <int XF, int WF, int S, int KSUB>
static inline bool gemm_ring_launch_t(const GemmParams& p, hipStream_t stream) {
  constexpr int BM = 32 * XF, BN = 32 * WF, LDS = S * KSUB * (BM + BN) * 128;
  static DeviceOnce once;
  const int dev = once.slot();
  if (once.need(dev)) {
    if (hipFuncSetAttribute((const void*)gemm_ring_kernel<XF, WF, S, KSUB>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    once.mark(dev);
  }
  const int64_t gy = ((int64_t)p.M + BM - 1) / BM, gx = ((int64_t)p.N + BN - 1) / BN;
  if (gy > 65535 || gx > 0x7fffffffLL || p.K % (64 * KSUB) != 0) return false;
  gemm_ring_kernel<XF, WF, S, KSUB><<<dim3((unsigned)gx, (unsigned)gy), 256, LDS, stream>>>(p);
  return true;
}
// Ring configurations (rows x weight rows per workgroup, stages, 64-wide k sub-tiles per stage):
//   0: 64x64 S3 K1   1: 64x64 S2 K2   2: 64x64 S3 K2   3: 32x64 S3 K2   4: 32x32 S3 K4
//   5: 32x64 S4 K1   6: 32x32 S4 K1
static inline bool gemm_ring_launch(const GemmParams& p, int shape, hipStream_t stream) {
  if (p.K % 64 != 0 || p.M <= 0 || p.N <= 0) return false;
  const int64_t lim = (int64_t)1 << 32;
  if (((int64_t)p.M * p.ldx + p.K) * 2 >= lim || ((int64_t)p.N * p.ldw + p.K) * 2 >= lim) return false;
  switch (shape) {
    case 0: return gemm_ring_launch_t<2, 2, 3, 1>(p, stream);
    case 1: return gemm_ring_launch_t<2, 2, 2, 2>(p, stream);
    case 2: return gemm_ring_launch_t<2, 2, 3, 2>(p, stream);
    case 3: return gemm_ring_launch_t<1, 2, 3, 2>(p, stream);
    case 4: return gemm_ring_launch_t<1, 1, 3, 4>(p, stream);
    case 5: return gemm_ring_launch_t<1, 2, 4, 1>(p, stream);
    case 6: return gemm_ring_launch_t<1, 1, 4, 1>(p, stream);
    default: return false;
  }
}

// Picks the ring configuration for a decode-sized batch (measured on M = 1 .. 512 against the
// qkv / o / router projections of the 30B-A3B shape and N up to 8192): enough workgroups to occupy every CU
// first, then the largest tile (least L2 -> LDS traffic), then fewer, longer steps when K allows. The 32x32
// configuration holds 96 KB of LDS, so one workgroup per CU: past 256 of them the 32x64 one is faster.
static inline bool gemm_ring_auto(const GemmParams& p, hipStream_t stream) {
  const int64_t m64 = (p.M + 63) / 64, m32 = (p.M + 31) / 32;
  const int64_t n64 = (p.N + 63) / 64, n32 = (p.N + 31) / 32;
  const bool k2 = p.K % 128 == 0, k4 = p.K % 256 == 0;
  int shape;
  if (m64 * n64 >= 512) shape = 0;
  else if (m64 * n64 >= 300) shape = k2 ? 1 : 0;
  else if (m64 * n64 >= 200) shape = k2 ? 2 : 0;
  else if (m32 * n64 >= 200) shape = k2 ? 3 : 5;
  else if (m32 * n32 > 256 && m32 * n64 >= 128) shape = k2 ? 3 : 5;
  else shape = k4 ? 4 : 6;
  return gemm_ring_launch(p, shape, stream);
}

}  // namespace vx
