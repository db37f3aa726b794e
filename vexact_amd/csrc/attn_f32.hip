// Kernels of the fp32 attention path: thread index -> (row, head), the arithmetic is attn_f32.h.
#include "attn_f32_launch.h"

namespace vx {

__global__ __launch_bounds__(256) void attn_f32_forward_kernel(AttnF32 p, int64_t n) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx < n) attn_f32_forward_row(p, (int)(idx / p.Hq), (int)(idx % p.Hq));
}

__global__ __launch_bounds__(256) void attn_f32_delta_kernel(AttnF32Bwd p, int64_t n) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx < n) attn_f32_delta_row(p, (int)(idx / p.Hq), (int)(idx % p.Hq));
}

__global__ __launch_bounds__(256) void attn_f32_dq_kernel(AttnF32Bwd p, int64_t n) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx < n) attn_f32_dq_row(p, (int)(idx / p.Hq), (int)(idx % p.Hq));
}

__global__ __launch_bounds__(256) void attn_f32_dkv_kernel(AttnF32Bwd p, int64_t n) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx < n) attn_f32_dkv_row(p, (int)(idx / p.Hkv), (int)(idx % p.Hkv));
}

static inline bool grid_for(int64_t n, unsigned& blocks) {
  const int64_t b = (n + 255) / 256;
  if (b <= 0 || b > 0x7fffffffLL) return false;
  blocks = (unsigned)b;
  return true;
}

int launch_attn_f32_forward(const AttnF32& p, int64_t total_q, hipStream_t stream) {
  unsigned blocks;
  if (total_q > 0x7fffffffLL || !grid_for(total_q * p.Hq, blocks)) return VX_ERR_UNSUPPORTED;
  attn_f32_forward_kernel<<<blocks, 256, 0, stream>>>(p, total_q * p.Hq);
  return launch_status();
}

int launch_attn_f32_backward(const AttnF32Bwd& p, int64_t total_q, int64_t total_k, hipStream_t stream) {
  unsigned bq, bk;
  if (total_q > 0x7fffffffLL || total_k > 0x7fffffffLL) return VX_ERR_UNSUPPORTED;
  if (!grid_for(total_q * p.Hq, bq) || !grid_for(total_k * p.Hkv, bk)) return VX_ERR_UNSUPPORTED;
  attn_f32_delta_kernel<<<bq, 256, 0, stream>>>(p, total_q * p.Hq);
  attn_f32_dq_kernel<<<bq, 256, 0, stream>>>(p, total_q * p.Hq);
  attn_f32_dkv_kernel<<<bk, 256, 0, stream>>>(p, total_k * p.Hkv);
  return launch_status();
}

}  // namespace vx
