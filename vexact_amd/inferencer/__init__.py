"""Import paths of the reference's ``vexact.inferencer`` package for the parts rebuilt here."""

from .sampler import Sampler

__all__ = ["Sampler"]
