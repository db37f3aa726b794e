// Dense GEMM entry points.
//   vx_gemm_bf16_nt : C = X * W^T (+bias), bf16, both operands K-contiguous (the nn.Linear case)
//   vx_gemm_generic : any strides, f32 / bf16 / f16 - one thread per output element, K walked in
//                     ascending order with fp32 FMAs; used for layouts the fast path rejects
//   vx_transpose_bf16 : packs a [K, N] row-major operand to [N, K] so it can use the fast path
// Replaces matmul_kernel_persistent / matmul_persistent
// (vexact/batch_invariant_ops/batch_invariant_ops.py:53-228) and _bmm_kernel / triton_bmm (:484-606).
#include "gemm_core.h"
#include "gemm_wide.h"

namespace vx {

template <typename T> struct Cvt;
template <> struct Cvt<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct Cvt<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = f32_to_bf16(v); }
};
template <> struct Cvt<_Float16> {
  static __device__ __forceinline__ float ld(const _Float16* p) { return (float)*p; }
  static __device__ __forceinline__ void st(_Float16* p, float v) { *p = (_Float16)v; }
};

// Batched, fully strided. 16x16 thread tile: threadIdx.x walks n so stores coalesce.
template <typename T>
__global__ __launch_bounds__(256) void gemm_generic_kernel(
    const T* __restrict__ a, const T* __restrict__ b, const T* __restrict__ bias, T* __restrict__ c,
    int64_t M, int64_t N, int64_t K, int64_t sab, int64_t sam, int64_t sak, int64_t sbb, int64_t sbk,
    int64_t sbn, int64_t scb, int64_t scm, int64_t scn) {
  const int64_t n = (int64_t)blockIdx.x * 16 + (threadIdx.x & 15);
  const int64_t m = (int64_t)blockIdx.y * 16 + (threadIdx.x >> 4);
  const int64_t bt = blockIdx.z;
  if (m >= M || n >= N) return;
  const T* ap = a + bt * sab + m * sam;
  const T* bp = b + bt * sbb + n * sbn;
  float acc = 0.f;
  for (int64_t k = 0; k < K; k++) acc = fmaf(Cvt<T>::ld(ap + k * sak), Cvt<T>::ld(bp + k * sbk), acc);
  if (bias) acc += Cvt<T>::ld(bias + n);
  Cvt<T>::st(c + bt * scb + m * scm + n * scn, acc);
}

// out[n, k] = in[k, n]; 64x64 tiles through LDS
__global__ __launch_bounds__(256) void transpose_bf16_kernel(const bf16_t* __restrict__ in,
                                                            bf16_t* __restrict__ out, int64_t K,
                                                            int64_t N, int64_t ldi, int64_t ldo) {
  __shared__ bf16_t t[64][66];
  const int64_t k0 = (int64_t)blockIdx.y * 64, n0 = (int64_t)blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4)
    if (k0 + r < K && n0 + tx < N) t[r][tx] = in[(k0 + r) * ldi + n0 + tx];
  __syncthreads();
  for (int r = ty; r < 64; r += 4)
    if (n0 + r < N && k0 + tx < K) out[(n0 + r) * ldo + k0 + tx] = t[tx][r];
}

}  // namespace vx

using namespace vx;

extern "C" {

int vx_gemm_bf16_nt(const void* x, const void* w, const void* bias, void* c, int64_t M, int64_t N,
                    int64_t K, int64_t ldx, int64_t ldw, int64_t ldc, hipStream_t stream) {
  if (!x || !w || !c || M < 0 || N <= 0 || K <= 0) return VX_ERR_ARG;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return VX_ERR_ARG;
  if (!gemm_fast_ok(x, w, K, ldx, ldw)) return VX_ERR_UNSUPPORTED;
  if (M == 0) return VX_OK;
  GemmParams p = {};
  p.x = (const bf16_t*)x; p.ldx = ldx;
  p.w = (const bf16_t*)w; p.ldw = ldw;
  p.bias = (const bf16_t*)bias;
  p.c = (bf16_t*)c; p.ldc = ldc;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  // Kernel choice (any choice gives the same bits): up to 512 rows the weight-streaming kernel wins
  // unless the problem is large enough to fill the chip with 128x128 tiles; its row-tile height is
  // the largest of 64 / 32 / 16 that still yields >= 256 workgroups.
  const int64_t nt = (N + 63) / 64;
  int mt = 0;
  if (M <= 16) mt = 1;
  else if (M <= 32) mt = 2;
  else if (M <= 64) mt = 4;
  else if (M <= 512 && nt * ((M + 63) / 64) <= 1024) {
    mt = 1;
    if (nt * ((M + 63) / 64) >= 256) mt = 4;
    else if (nt * ((M + 31) / 32) >= 256) mt = 2;
  }
  // 65 .. 512 rows: the LDS ring kernel, whose loads do not wait on one wavefront's MFMA chain. Up to 64 rows
  // too when the weight matrix is small (N <= 8192): the streaming kernel then has at most 128 workgroups of
  // dependent loads (o projection at 16 rows: 20.0 us, ring 10.8 us; router 10.9 -> 5.8; equal near N = 16384,
  // streaming ahead from N = 32768 on).
  if (mt != 0 && (M > 64 || nt <= 128) && gemm_ring_auto(p, stream)) return launch_status();
  if (mt != 0) {
    const dim3 grid((unsigned)nt, (unsigned)((M + 16 * mt - 1) / (16 * mt)));
    // up to 32 rows: 32 KB activation chunks (more workgroups per CU; lm_head at 1 / 7 / 16 / 32 rows 114 -> 111,
    // 114 -> 112, 115 -> 113, 125 -> 121 us); at 64 rows the 64 KB chunks are ahead (136 against 139 us)
    if (mt == 1) gemm_stream_kernel<1, EPI_PLAIN, false, 8, 2><<<grid, 256, 0, stream>>>(p);
    else if (mt == 2) gemm_stream_kernel<2, EPI_PLAIN, false, 8, 2><<<grid, 256, 0, stream>>>(p);
    else gemm_stream_kernel<4, EPI_PLAIN, false><<<grid, 256, 0, stream>>>(p);
  } else {
    // 513 .. 1024 rows against a moderate weight matrix: still the ring kernel (64 x 64 tiles, three stages). Measured
    // against the 128 x 128 tiles that ran here: o projection (2048 x 4096) at 513 / 1024 rows 61 -> 26 / 62 -> 29 us,
    // q/k/v (5120 x 2048) 35 -> 23 / 46 -> 35 us; a 12288 x 4096 matrix is level at 384 rows and 27 % behind at 512,
    // hence the bound on tiles x depth.
    if (M <= 1024 && K % 64 == 0 && nt * ((M + 63) / 64) * K <= ((int64_t)1 << 22) && gemm_ring_launch(p, 0, stream))
      return launch_status();
    // many rows: 256x256 tiles once they fill at least half the chip, else 128x128 tiles
    const int64_t wide_tiles = ((M + WD_BM - 1) / WD_BM) * ((N + WD_BN - 1) / WD_BN);
    if (wide_tiles >= 128 && gemm_wide_launch(p, stream)) return launch_status();
    // many rows but few columns (router logits over a prefill chunk): the 64x64 ring kernel yields four
    // times the workgroups of the 128x128 tiles
    if (N <= 256 && ((M + 127) / 128) * ((N + 127) / 128) < 256 && gemm_ring_launch(p, 0, stream)) return launch_status();
    const int64_t mtl = (M + TL_BM - 1) / TL_BM;
    if (mtl > 65535) return VX_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)((N + TL_BN - 1) / TL_BN), (unsigned)mtl);
    gemm_tiled_kernel<EPI_PLAIN, false><<<grid, 256, 0, stream>>>(p);
  }
  return launch_status();
}

// Dense SwiGLU: C[M, N] = r16(r16(silu(r16(X Wg^T))) * r16(X Wu^T)), both projections and the
// activation in one kernel. kind < 0: automatic; 0 / 1 / 3 force the streaming (mt rows / 16), the
// 128x128 tiled or the 256x256 wide kernel (for the tests that check they agree bit for bit).
static int gemm_swiglu_dispatch(const GemmParams& p, int kind, int mt, hipStream_t stream) {
  const int64_t M = p.M, N = p.N;
  if (kind < 0) {
    const int64_t wide_tiles = ((M + WD_BM - 1) / WD_BM) * ((N + 127) / 128);
    if (M <= 16) { kind = 0; mt = 1; }
    else if (M <= 32) { kind = 0; mt = 2; }
    else if (M <= 64) { kind = 0; mt = 4; }
    else if (M > 384 && wide_tiles >= 64 && p.K % WD_BK == 0) kind = 3;  // measured crossover
    else kind = 1;
  }
  if (kind == 0) {
    if (mt != 1 && mt != 2 && mt != 4) return VX_ERR_ARG;
    const int64_t my = (M + 16 * mt - 1) / (16 * mt);
    if (my > 65535) return VX_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)((N + 63) / 64), (unsigned)my);
    if (mt == 1) gemm_stream_kernel<1, EPI_SWIGLU, false><<<grid, 256, 0, stream>>>(p);
    else if (mt == 2) gemm_stream_kernel<2, EPI_SWIGLU, false><<<grid, 256, 0, stream>>>(p);
    else gemm_stream_kernel<4, EPI_SWIGLU, false><<<grid, 256, 0, stream>>>(p);
  } else if (kind == 1) {
    const int64_t my = (M + TL_BM - 1) / TL_BM;
    if (my > 65535) return VX_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)((N + 63) / 64), (unsigned)my);
    gemm_tiled_kernel<EPI_SWIGLU, false><<<grid, 256, 0, stream>>>(p);
  } else if (kind == 3) {
    if (!gemm_wide_swiglu_launch(p, stream)) return VX_ERR_UNSUPPORTED;
  } else {
    return VX_ERR_ARG;
  }
  return launch_status();
}

int vx_gemm_swiglu_bf16_nt(const void* x, const void* w_gate, const void* w_up, void* c, int64_t M, int64_t N,
                           int64_t K, int64_t ldx, int64_t ldw, int64_t ldc, int kind, int mt, hipStream_t stream) {
  if (!x || !w_gate || !w_up || !c || M < 0 || N <= 0 || K <= 0) return VX_ERR_ARG;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return VX_ERR_ARG;
  if (!gemm_fast_ok(x, w_gate, K, ldx, ldw) || !gemm_fast_ok(x, w_up, K, ldx, ldw)) return VX_ERR_UNSUPPORTED;
  if (M == 0) return VX_OK;
  GemmParams p = {};
  p.x = (const bf16_t*)x; p.ldx = ldx;
  p.w = (const bf16_t*)w_gate; p.w2 = (const bf16_t*)w_up; p.ldw = ldw;
  p.c = (bf16_t*)c; p.ldc = ldc;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  return gemm_swiglu_dispatch(p, kind, mt, stream);
}

// Forces one kernel regardless of M (kind 0 = streaming with 16*mt rows per tile, mt in {1,2,4};
// kind 1 = 128x128 tiled; kind 2 = streaming, 16 k-steps in flight; kind 3 = 256x256 wide tiles,
// needs K % 64 == 0; kind 4 = LDS ring kernel, mt = configuration 0..6). For tests that check
// that all kernels give the same bits.
int vx_gemm_bf16_nt_variant(const void* x, const void* w, const void* bias, void* c, int64_t M,
                            int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldc, int kind,
                            int mt, hipStream_t stream) {
  if (!x || !w || !c || M <= 0 || N <= 0 || K <= 0) return VX_ERR_ARG;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return VX_ERR_ARG;
  if (!gemm_fast_ok(x, w, K, ldx, ldw)) return VX_ERR_UNSUPPORTED;
  GemmParams p = {};
  p.x = (const bf16_t*)x; p.ldx = ldx;
  p.w = (const bf16_t*)w; p.ldw = ldw;
  p.bias = (const bf16_t*)bias;
  p.c = (bf16_t*)c; p.ldc = ldc;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  if (kind == 0) {
    if (mt != 1 && mt != 2 && mt != 4) return VX_ERR_ARG;
    const int64_t bm = 16 * mt;
    const int64_t my = (M + bm - 1) / bm;
    if (my > 65535) return VX_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)((N + 63) / 64), (unsigned)my);
    if (mt == 1) gemm_stream_kernel<1, EPI_PLAIN, false><<<grid, 256, 0, stream>>>(p);
    else if (mt == 2) gemm_stream_kernel<2, EPI_PLAIN, false><<<grid, 256, 0, stream>>>(p);
    else gemm_stream_kernel<4, EPI_PLAIN, false><<<grid, 256, 0, stream>>>(p);
  } else if (kind == 2) {  // streaming with 16 k-steps in flight
    if (mt != 1 && mt != 2 && mt != 4) return VX_ERR_ARG;
    const int64_t bm = 16 * mt;
    const int64_t my = (M + bm - 1) / bm;
    if (my > 65535) return VX_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)((N + 63) / 64), (unsigned)my);
    if (mt == 1) gemm_stream_kernel<1, EPI_PLAIN, false, 16><<<grid, 256, 0, stream>>>(p);
    else if (mt == 2) gemm_stream_kernel<2, EPI_PLAIN, false, 16><<<grid, 256, 0, stream>>>(p);
    else gemm_stream_kernel<4, EPI_PLAIN, false, 16><<<grid, 256, 0, stream>>>(p);
  } else if (kind == 1) {
    const int64_t my = (M + TL_BM - 1) / TL_BM;
    if (my > 65535) return VX_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)((N + TL_BN - 1) / TL_BN), (unsigned)my);
    gemm_tiled_kernel<EPI_PLAIN, false><<<grid, 256, 0, stream>>>(p);
  } else if (kind == 3) {  // wide 256x256 tiles
    if (!gemm_wide_launch(p, stream)) return VX_ERR_UNSUPPORTED;
  } else if (kind == 4) {  // LDS ring, mt = tile shape code
    if (!gemm_ring_launch(p, mt, stream)) return VX_ERR_UNSUPPORTED;
  } else {
    return VX_ERR_ARG;
  }
  return launch_status();
}

int vx_gemm_generic(const void* a, const void* b, const void* bias, void* c, int dtype, int64_t batch,
                    int64_t M, int64_t N, int64_t K, int64_t sab, int64_t sam, int64_t sak,
                    int64_t sbb, int64_t sbk, int64_t sbn, int64_t scb, int64_t scm, int64_t scn,
                    hipStream_t stream) {
  if (!a || !b || !c || batch < 0 || M < 0 || N < 0 || K < 0) return VX_ERR_ARG;
  if (batch == 0 || M == 0 || N == 0) return VX_OK;
  const int64_t gx = (N + 15) / 16, gy = (M + 15) / 16;
  if (gx > 0x7fffffffLL || gy > 65535 || batch > 65535) return VX_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)batch);
  switch (dtype) {
    case 0:
      gemm_generic_kernel<float><<<grid, 256, 0, stream>>>((const float*)a, (const float*)b,
                                                           (const float*)bias, (float*)c, M, N, K,
                                                           sab, sam, sak, sbb, sbk, sbn, scb, scm, scn);
      break;
    case 1:
      gemm_generic_kernel<bf16_t><<<grid, 256, 0, stream>>>(
          (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)bias, (bf16_t*)c, M, N, K, sab, sam,
          sak, sbb, sbk, sbn, scb, scm, scn);
      break;
    case 2:
      gemm_generic_kernel<_Float16><<<grid, 256, 0, stream>>>(
          (const _Float16*)a, (const _Float16*)b, (const _Float16*)bias, (_Float16*)c, M, N, K, sab,
          sam, sak, sbb, sbk, sbn, scb, scm, scn);
      break;
    default: return VX_ERR_UNSUPPORTED;
  }
  return launch_status();
}

int vx_transpose_bf16(const void* in, void* out, int64_t K, int64_t N, int64_t ld_in, int64_t ld_out,
                      hipStream_t stream) {
  if (!in || !out || K < 0 || N < 0) return VX_ERR_ARG;
  if (K == 0 || N == 0) return VX_OK;
  const int64_t gx = (N + 63) / 64, gy = (K + 63) / 64;
  if (gx > 0x7fffffffLL || gy > 65535) return VX_ERR_UNSUPPORTED;
  transpose_bf16_kernel<<<dim3((unsigned)gx, (unsigned)gy), 256, 0, stream>>>(
      (const bf16_t*)in, (bf16_t*)out, K, N, ld_in, ld_out);
  return launch_status();
}

}  // extern "C"
