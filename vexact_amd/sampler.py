"""``Sampler`` with the reference's interface (vexact/inferencer/sampler.py:29-113) over the HIP
sampling kernel.

Differences from the reference, all on purpose:

* top-k / top-p / sampling run in one kernel without sorting the vocabulary and without
  materialising softmax, cumulative-sum or noise tensors;
* every sampled row is keyed by (seed, position): requests that carry ``seed`` use it together with
  ``sampling_positions`` (repeatable and request-order invariant, no vLLM needed); requests without a
  seed get one drawn per row from torch's default CPU generator, so ``torch.manual_seed`` makes a
  run repeatable, as with the reference's ``exponential_``;
* equal logits are kept or masked together by top-p.
"""

from __future__ import annotations

from typing import Optional, Sequence

import torch
from torch import Tensor

from . import ops


class Sampler:
    @torch.inference_mode()
    def batch_sample_token(
        self,
        batched_logits: Tensor,
        gen_configs: Sequence,
        sampling_positions: Optional[Tensor] = None,
    ) -> Tensor:
        """Next token for each row of ``batched_logits`` [batch, vocab]. As in the reference, k, p and
        the temperature of the first config apply to the whole batch."""
        cfg = gen_configs[0]
        k, p = cfg.top_k, cfg.top_p
        assert p is not None, "top_p must be set (use 1.0 to disable)"
        if k is not None and int(k) <= 0:
            k = None
        temp = cfg.temperature
        do_sample = bool(cfg.do_sample) and temp > 0 and float(p) > 0
        if not do_sample:
            _, tokens = ops.logprobs(batched_logits, None, return_tokens=True)  # first argmax
            return tokens
        device = batched_logits.device
        B = batched_logits.shape[0]
        seeds = [getattr(c, "seed", None) for c in gen_configs]
        has_seed = [s is not None for s in seeds]
        if any(has_seed):
            if not all(has_seed):
                raise ValueError("Seeded sampling requires every request in the batch to set seed.")
            if sampling_positions is None:
                raise ValueError("sampling_positions must be set for seeded sampling.")
            seed_t = torch.tensor([int(s) for s in seeds], dtype=torch.int64).to(device)
            pos_t = sampling_positions.to(device=device, dtype=torch.int64).contiguous()
        else:
            seed_t = torch.randint(0, 2**62, (B,), dtype=torch.int64).to(device)
            pos_t = torch.zeros(B, dtype=torch.int64, device=device)
        if batched_logits.dtype not in (torch.bfloat16, torch.float32):
            batched_logits = batched_logits.to(torch.float32)
        return ops.sample_tokens(batched_logits, float(temp), k, float(p), seed_t, pos_t)
