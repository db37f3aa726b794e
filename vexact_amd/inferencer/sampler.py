"""``vexact.inferencer.sampler`` import path: the sampler lives in ``vexact_amd.sampler``."""

from ..sampler import Sampler

__all__ = ["Sampler"]
