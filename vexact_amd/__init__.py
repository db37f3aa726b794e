"""vexact_amd: MI355X (gfx950) kernels for VeXact's batch-invariant inference hot path.

``vexact_amd.batch_invariant_ops`` mirrors ``vexact.batch_invariant_ops`` name for name; the
arithmetic lives in ``libvexact_hip.so`` (hand-written HIP, C ABI in ``include/vexact_hip.h``).
"""

__version__ = "0.1.0"
