"""Compile the HIP kernels into ``libvexact_hip.so`` (gfx950 only, no torch dependency).

The library is built in-tree so that it travels with the source snapshot to the GPU machine;
nothing here needs a GPU: hipcc cross-compiles.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libvexact_hip.so")
SOURCES = ["row_ops.hip", "gemm.hip", "gemm_other.hip", "paged_attn.hip", "paged_attn_pad.hip", "paged_attn_f16.hip", "attn_bwd.hip", "attn_bwd_f16.hip", "attn_f32.hip", "moe.hip", "moe_bwd.hip", "glue.hip", "sampler.hip", "host_meta.cpp"]
HEADERS = ["common.h", "gemm_core.h", "gemm_wide.h", "attn_core.h", "attn_bwd_core.h", "attn_f32.h", "attn_f32_launch.h"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -ffp-contract=off: kernels that must agree bit for bit share source-level expressions, so the
# compiler may not fuse a*b+c differently from one kernel to the next.
# packed-fp32 ops are disabled on purpose (some forms are unreliable on the target machines).
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _compile_one(src: str, obj_dir: str) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    if src.endswith(".cpp"):  # host-only code: plain C++, no device pass
        cmd = [HIPCC, "-x", "c++", "-O3", "-std=c++17", "-fPIC", "-c", os.path.join(CSRC, src), "-o", obj]
    else:
        cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stderr[-4000:]}")
    return obj


def needs_build() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(os.path.join(CSRC, f)) > t for f in SOURCES + HEADERS)


def build(force: bool = True, verbose: bool = True) -> str:
    """Compile every kernel file and link the shared library. Returns its path."""
    if not force and not needs_build():
        return LIB_PATH
    obj_dir = os.path.join(CSRC, "build")
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 4)) as ex:
        objs = list(ex.map(lambda s: _compile_one(s, obj_dir), SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr[-4000:]}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH) // 1024} KiB)", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build()
