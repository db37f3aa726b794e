// fp16 attention backward: the register-form kernels of attn_bwd_core.h. A translation unit of its own for compile time.
#include "attn_bwd_core.h"

namespace vx {

int launch_attn_bwd_f16(const AttnBwdParams& p, int Db, int64_t total_q, int num_seqs, int max_q, int max_k, hipStream_t stream) {
  if (Db == 64) return launch_attn_bwd_generic<ElemF16, 64, true>(p, total_q, num_seqs, max_q, max_k, stream);
  if (Db == 128) return launch_attn_bwd_generic<ElemF16, 128, true>(p, total_q, num_seqs, max_q, max_k, stream);
  if (Db == 256) return launch_attn_bwd_generic<ElemF16, 256, true>(p, total_q, num_seqs, max_q, max_k, stream);
  return VX_ERR_UNSUPPORTED;
}

}  // namespace vx
