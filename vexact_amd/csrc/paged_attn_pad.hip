// Attention kernels (attn_core.h) for bf16 on head sizes between the built-for ones, or on rows that are not 16-byte addressable. A translation unit of its own for compile time.
#include "attn_core.h"

namespace vx {

int launch_attn_bf16_padded(const AttnParams& p, int DKb, int DVb, int mode, int max_q, int total_q, hipStream_t stream) {
  if (DKb == 64 && DVb == 64) return launch_attn<ElemBF16, 64, 64, true>(p, mode, max_q, total_q, stream);
  if (DKb == 128 && DVb == 128) return launch_attn<ElemBF16, 128, 128, true>(p, mode, max_q, total_q, stream);
  if (DKb == 256 && DVb == 128) return launch_attn<ElemBF16, 256, 128, true>(p, mode, max_q, total_q, stream);
  if (DKb == 256 && DVb == 256) return launch_attn<ElemBF16, 256, 256, true>(p, mode, max_q, total_q, stream);
  return VX_ERR_UNSUPPORTED;
}

}  // namespace vx
