// Launchers of the fp32 attention kernels (attn_f32.hip) for the entry points in paged_attn.hip and attn_bwd.hip.
#pragma once
#include "attn_f32.h"
#include "common.h"

namespace vx {

// one thread per (query row, head); any mode (paged decode / general, packed)
int launch_attn_f32_forward(const AttnF32& p, int64_t total_q, hipStream_t stream);
// delta, then dQ (one thread per query row and head) and dK / dV (one thread per key row and kv head)
int launch_attn_f32_backward(const AttnF32Bwd& p, int64_t total_q, int64_t total_k, hipStream_t stream);

}  // namespace vx
