// fp16 and fp32 "NT" GEMM on the matrix cores: C[m, n] = cast(sum_k X[m, k] W[n, k] (+ bias[n])), X and W
// K-contiguous (the nn.Linear case), fp32 accumulate, K ascending, no split-K.
// Replaces the fp16 / fp32 configurations of matmul_kernel_persistent
// (vexact/batch_invariant_ops/batch_invariant_ops.py:53-131, tile table :182-206). The reference lets tl.dot
// take its default for fp32 inputs (TF32 on its hardware); here fp32 products are true fp32
// (v_mfma_f32_16x16x4_f32).
//
// ONE kernel and one tile shape for every M: a 256-thread workgroup computes 64 activation rows x 64 weight
// rows, 32 k per step through LDS; wavefront (wm, wn) of the 2 x 2 arrangement owns activation rows
// [32 wm, +32) and weight rows [32 wn, +32). As in the bf16 kernels the weight fragment is the MFMA A operand
// and the activation fragment the B operand, and every output element is one accumulator chain over K, so a
// row's result cannot depend on the other rows of the call. Rows and k past the ends are zero filled.
#include "common.h"

namespace vx {

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

constexpr int GO_BM = 64, GO_BN = 64, GO_BK = 32;

template <typename T> struct GoType;
template <> struct GoType<float> {
  static constexpr int PAD = 4;  // row pitch 36 floats: the 16 rows of a fragment read hit distinct banks
  static __device__ __forceinline__ float to_f32(float v) { return v; }
  static __device__ __forceinline__ float from_f32(float v) { return v; }
};
template <> struct GoType<_Float16> {
  static constexpr int PAD = 8;
  static __device__ __forceinline__ float to_f32(_Float16 v) { return (float)v; }
  static __device__ __forceinline__ _Float16 from_f32(float v) { return (_Float16)v; }
};

// VEC: rows are 16-byte aligned and K is a multiple of the 16-byte vector, so a thread moves 16 bytes at a time
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void gemm_other_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                         const T* __restrict__ bias, T* __restrict__ c, int M, int N,
                                                         int K, int64_t ldx, int64_t ldw, int64_t ldc) {
  constexpr int PITCH = GO_BK + GoType<T>::PAD;
  constexpr int VE = 16 / (int)sizeof(T);  // elements per 16-byte vector
  __shared__ __attribute__((aligned(16))) T xs[GO_BM * PITCH];
  __shared__ __attribute__((aligned(16))) T ws[GO_BN * PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * GO_BM, n0 = blockIdx.x * GO_BN;

  f32x4 acc[2][2];  // [activation tile i][weight tile j]
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int k0 = 0; k0 < K; k0 += GO_BK) {
    // ---- stage a 64 x 32 tile of each operand (zero filled past the ends)
    if constexpr (VEC) {
      constexpr int VPR = GO_BK / VE;                 // vectors per tile row
      constexpr int PER = GO_BM * VPR / 256;          // vectors per thread and operand
#pragma unroll
      for (int q = 0; q < PER; q++) {
        const int v = tid + 256 * q, row = v / VPR, col = (v % VPR) * VE;
        const bool kin = k0 + col < K;
        uint4 xv = make_uint4(0, 0, 0, 0), wv = make_uint4(0, 0, 0, 0);
        if (kin && m0 + row < M) xv = *(const uint4*)(x + (int64_t)(m0 + row) * ldx + k0 + col);
        if (kin && n0 + row < N) wv = *(const uint4*)(w + (int64_t)(n0 + row) * ldw + k0 + col);
        *(uint4*)(xs + row * PITCH + col) = xv;
        *(uint4*)(ws + row * PITCH + col) = wv;
      }
    } else {
      for (int e = tid; e < GO_BM * GO_BK; e += 256) {
        const int row = e / GO_BK, col = e % GO_BK;
        const bool kin = k0 + col < K;
        xs[row * PITCH + col] = (kin && m0 + row < M) ? x[(int64_t)(m0 + row) * ldx + k0 + col] : (T)0;
        ws[row * PITCH + col] = (kin && n0 + row < N) ? w[(int64_t)(n0 + row) * ldw + k0 + col] : (T)0;
      }
    }
    __syncthreads();
    // ---- products, k ascending
    if constexpr (sizeof(T) == 2) {
      // one v_mfma_f32_16x16x32_f16 per tile pair: lane (r16, g) supplies row r16, k 8 g .. 8 g + 7
      f16x8 a[2], b[2];
#pragma unroll
      for (int j = 0; j < 2; j++) a[j] = *(const f16x8*)(ws + (32 * wn + 16 * j + r16) * PITCH + 8 * g);
#pragma unroll
      for (int i = 0; i < 2; i++) b[i] = *(const f16x8*)(xs + (32 * wm + 16 * i + r16) * PITCH + 8 * g);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j], b[i], acc[i][j], 0, 0, 0);
    } else {
      // eight v_mfma_f32_16x16x4_f32 per tile pair: lane (r16, g) supplies row r16, k 4 s + g of sub-step s
#pragma unroll
      for (int s = 0; s < GO_BK / 4; s++) {
        float a[2], b[2];
#pragma unroll
        for (int j = 0; j < 2; j++) a[j] = ws[(32 * wn + 16 * j + r16) * PITCH + 4 * s + g];
#pragma unroll
        for (int i = 0; i < 2; i++) b[i] = xs[(32 * wm + 16 * i + r16) * PITCH + 4 * s + g];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], b[i], acc[i][j], 0, 0, 0);
      }
    }
    __syncthreads();
  }

  // ---- lane holds C[m0 + 32 wm + 16 i + r16][n0 + 32 wn + 16 j + 4 g + r]
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int m = m0 + 32 * wm + 16 * i + r16;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int nb = n0 + 32 * wn + 16 * j + 4 * g;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int n = nb + r;
        if (n < N) {
          float v = acc[i][j][r];
          if (bias) v += GoType<T>::to_f32(bias[n]);
          c[(int64_t)m * ldc + n] = GoType<T>::from_f32(v);
        }
      }
    }
  }
}

template <typename T>
static int gemm_other_launch(const void* x, const void* w, const void* bias, void* c, int64_t M, int64_t N, int64_t K,
                             int64_t ldx, int64_t ldw, int64_t ldc, hipStream_t stream) {
  const int64_t gx = (N + GO_BN - 1) / GO_BN, gy = (M + GO_BM - 1) / GO_BM;
  if (gx > 0x7fffffffLL || gy > 65535) return VX_ERR_UNSUPPORTED;
  constexpr int VE = 16 / (int)sizeof(T);
  const bool vec = K % VE == 0 && ldx % VE == 0 && ldw % VE == 0 && ((uintptr_t)x | (uintptr_t)w) % 16 == 0;
  const dim3 grid((unsigned)gx, (unsigned)gy);
  if (vec)
    gemm_other_kernel<T, true><<<grid, 256, 0, stream>>>((const T*)x, (const T*)w, (const T*)bias, (T*)c, (int)M, (int)N,
                                                          (int)K, ldx, ldw, ldc);
  else
    gemm_other_kernel<T, false><<<grid, 256, 0, stream>>>((const T*)x, (const T*)w, (const T*)bias, (T*)c, (int)M, (int)N,
                                                           (int)K, ldx, ldw, ldc);
  return launch_status();
}

}  // namespace vx

using namespace vx;

extern "C" {

// dtype: 0 = float32, 2 = float16 (the codes of vx_gemm_generic; bf16 has its own entry points)
int vx_gemm_nt_mfma(const void* x, const void* w, const void* bias, void* c, int dtype, int64_t M, int64_t N, int64_t K,
                    int64_t ldx, int64_t ldw, int64_t ldc, hipStream_t stream) {
  if (!x || !w || !c || M < 0 || N <= 0 || K <= 0) return VX_ERR_ARG;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff || ldx < K || ldw < K || ldc < N) return VX_ERR_ARG;
  if (M == 0) return VX_OK;
  if (dtype == 0) return gemm_other_launch<float>(x, w, bias, c, M, N, K, ldx, ldw, ldc, stream);
  if (dtype == 2) return gemm_other_launch<_Float16>(x, w, bias, c, M, N, K, ldx, ldw, ldc, stream);
  return VX_ERR_UNSUPPORTED;
}

}  // extern "C"
