// Attention kernels (attn_core.h) for fp16 (every head size goes through the padded code). A translation unit of its own for compile time.
#include "attn_core.h"

namespace vx {

int launch_attn_f16(const AttnParams& p, int DKb, int DVb, int mode, int max_q, int total_q, hipStream_t stream) {
  if (DKb == 64 && DVb == 64) return launch_attn<ElemF16, 64, 64, true>(p, mode, max_q, total_q, stream);
  if (DKb == 128 && DVb == 128) return launch_attn<ElemF16, 128, 128, true>(p, mode, max_q, total_q, stream);
  if (DKb == 256 && DVb == 128) return launch_attn<ElemF16, 256, 128, true>(p, mode, max_q, total_q, stream);
  if (DKb == 256 && DVb == 256) return launch_attn<ElemF16, 256, 256, true>(p, mode, max_q, total_q, stream);
  return VX_ERR_UNSUPPORTED;
}

}  // namespace vx
