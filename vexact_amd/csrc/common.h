// Shared device helpers for the gfx950 (CDNA4) kernels: bf16 conversion, the one MFMA
// instruction every matrix product goes through, and fixed-shape wavefront reductions.
//
// Batch-invariance rule used throughout: an output element is produced by one chain of
// v_mfma_f32_16x16x32_bf16 instructions that walks the contraction index in ascending
// 32-wide chunks, with the same (lane-group, slot) -> index mapping in every kernel. Tile
// shapes may differ between kernels because MFMA rows and columns never mix.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace vx {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef uint16_t bf16_t;  // storage type in global memory

constexpr int kWave = 64;

// "Done once per device" flag for host code that raises a kernel's dynamic-LDS limit before its first launch: the
// attribute belongs to the function as loaded on one device, and several host threads may launch the same kernel.
// slot() is the current device's index (-1 if it cannot be tracked: the caller then repeats the set-up each time).
struct DeviceOnce {
  std::atomic<unsigned char> done[64] = {};
  int slot() const {
    int d = -1;
    if (hipGetDevice(&d) != hipSuccess || d < 0 || d >= 64) return -1;
    return d;
  }
  bool need(int d) const { return d < 0 || !done[d].load(std::memory_order_acquire); }
  void mark(int d) { if (d >= 0) done[d].store(1, std::memory_order_release); }
};

// Status codes returned over the C ABI.
enum : int {
  VX_OK = 0,
  VX_ERR_ARG = -1,       // bad pointer / size / stride
  VX_ERR_UNSUPPORTED = -2,
  VX_ERR_WORKSPACE = -3,  // workspace too small
  VX_ERR_LAUNCH = -4,
};

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __builtin_bit_cast(float, (uint32_t)v << 16);
}
// round-to-nearest-even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  __bf16 h = (__bf16)f;
  return __builtin_bit_cast(bf16_t, h);
}
// both halves in one v_cvt_pk_bf16_f32 (same rounding as f32_to_bf16)
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ float bf16lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

// D(16x16) += A(16x32) * B(32x16). Lane l supplies A[row l%16][k 8*(l/16) .. +8) and
// B[k 8*(l/16) .. +8)][col l%16]; it receives D[4*(l/16) + r][l%16], r = 0..3.
__device__ __forceinline__ f32x4 mfma16(uint4 a, uint4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// The two 16-bit element types of the attention kernels: how eight of them enter the matrix core, how two fp32
// values round (to nearest even) into a packed pair, and how a packed pair widens again. Kernels take one of these
// as a template parameter; everything else (layouts, transposes, the order of every sum) is the same for both.
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
struct ElemBF16 {
  static constexpr int kDtype = 0;
  static __device__ __forceinline__ f32x4 mfma(uint4 a, uint4 b, f32x4 c) { return mfma16(a, b, c); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
  static __device__ __forceinline__ float lo(uint32_t w) { return bf16lo(w); }
  static __device__ __forceinline__ float hi(uint32_t w) { return bf16hi(w); }
  // acc + lo + hi of a packed pair in one v_dot2c_f32_bf16 against a pair of ones
  static __device__ __forceinline__ float add2(uint32_t pk, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pk), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), acc, false);
  }
};
struct ElemF16 {
  static constexpr int kDtype = 1;
  static __device__ __forceinline__ f32x4 mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
  }
  static __device__ __forceinline__ float lo(uint32_t w) { return (float)__builtin_bit_cast(f16x2_t, w)[0]; }
  static __device__ __forceinline__ float hi(uint32_t w) { return (float)__builtin_bit_cast(f16x2_t, w)[1]; }
  static __device__ __forceinline__ float add2(uint32_t pk, float acc) { return (acc + lo(pk)) + hi(pk); }
};

// 16-byte global loads. The address must always be dereferenceable (callers clamp it); zeroing
// is done on the loaded VALUE, and only where the value is consumed, so that a load stays a single
// global_load_dwordx4 and the wait for it is not pulled up to the issue point.
__device__ __forceinline__ uint4 ldg16_raw(const void* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ uint4 mask16(uint4 v, bool ok) {
  v.x = ok ? v.x : 0u;
  v.y = ok ? v.y : 0u;
  v.z = ok ? v.z : 0u;
  v.w = ok ? v.w : 0u;
  return v;
}
__device__ __forceinline__ uint4 ldg16(const void* p, bool ok) { return mask16(ldg16_raw(p), ok); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Block-wide sum over NW wavefronts through LDS; every thread gets the result. The order
// (lane butterfly, then wave 0..NW-1 ascending) is the same for any grid size.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red /* >= NW floats */) {
  v = wave_sum(v);
  if constexpr (NW == 1) return v;
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float s = red[0];
#pragma unroll
  for (int i = 1; i < NW; i++) s += red[i];
  return s;
}
template <int NW>
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  if constexpr (NW == 1) return v;
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float s = red[0];
#pragma unroll
  for (int i = 1; i < NW; i++) s = fmaxf(s, red[i]);
  return s;
}

// Direct-to-LDS loads (global memory -> LDS without staging registers). The LDS byte address of lane 0 goes into m0, the
// 64 lanes' pieces land behind it in lane order. Written as asm, not through __builtin_amdgcn_global_load_lds, on
// purpose: told that the instruction writes LDS, the compiler waits for it (vmcnt(0)) before the next LDS read it
// schedules, while the kernels keep several steps of these loads in flight and wait explicitly before the barrier that
// precedes their first use. Each statement sets m0 and consumes it in its own text and names m0 as clobbered; nothing
// else in these kernels lives in m0 (no indexed register arrays, no other LDS-DMA or message instructions), so the
// compiler's warning that a clobber of a reserved register is not saved and restored for the asm's sake does not bite.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
// 16 bytes per lane from (wave-uniform base in scalar registers) + (32-bit byte offset per lane)
__device__ __forceinline__ void lds_load16_sv(uint32_t lds_dst, uint32_t voff, const void* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(lds_dst), "v"(voff), "s"(sbase) : "memory", "m0");
}
// 16 bytes per lane from a full per-lane address
__device__ __forceinline__ void lds_load16_v(uint32_t lds_dst, const void* vaddr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(lds_dst), "v"(vaddr) : "memory", "m0");
}
// 4 bytes per lane from a full per-lane address
__device__ __forceinline__ void lds_load4_v(uint32_t lds_dst, const void* vaddr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" :: "s"(lds_dst), "v"(vaddr) : "memory", "m0");
}
#pragma clang diagnostic pop

// Reciprocal square root of the two RMSNorm forms. Form 0 is the reference kernel's 1 / sqrt(.) in fp32 (two
// roundings, batch_invariant_ops.py:653-660). Form 1 is what HuggingFace's module computes with torch.rsqrt on this
// device: measured on the GPU over 2^24 arguments, torch.rsqrt(x) has the bits of the double-precision quotient
// 1 / sqrt(x) rounded to fp32 once, whereas fp32 1 / sqrt and the hardware's approximate rsq differ from it in 25 %
// and 11 % of the arguments. A fused kernel in that form must give the bits of the module's own tensor operations.
// Once per row and thread, so the double-precision operations do not show in the run time.
__device__ __forceinline__ float rms_inv(float mean_sq_eps, int mode) {
  return mode == 0 ? 1.0f / sqrtf(mean_sq_eps) : (float)(1.0 / sqrt((double)mean_sq_eps));
}

static inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? VX_OK : VX_ERR_LAUNCH;
}

}  // namespace vx
