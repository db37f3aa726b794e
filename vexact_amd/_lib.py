"""ctypes binding of ``libvexact_hip.so`` (the C ABI declared in ``include/vexact_hip.h``).

There is deliberately no CPU fallback: if the library is missing, every op raises.
"""

from __future__ import annotations

import ctypes
import os
import threading

from ._build import LIB_PATH

_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float

# name -> (restype, argtypes); order follows include/vexact_hip.h
PROTOTYPES = {
    "vx_abi_version": (_I, []),
    "vx_status_string": (ctypes.c_char_p, [_I]),
    "vx_mean_dim": (_I, [_P, _P, _I, _L, _L, _L, _L, _L, _L, _L, _L, _P]),
    "vx_rms_norm": (_I, [_P, _P, _P, _P, _P, _I, _L, _L, _L, _L, _L, _L, _F, _I, _P]),
    "vx_log_softmax_workspace_bytes": (_L, [_L, _L]),
    "vx_log_softmax": (_I, [_P, _P, _I, _L, _L, _L, _L, _P, _L, _P]),
    "vx_logprobs": (_I, [_P, _P, _P, _P, _I, _L, _L, _L, _P, _L, _P]),
    "vx_logprobs_static": (_I, [_P, _P, _P, _P, _I, _L, _L, _L, _P]),
    "vx_gemm_bf16_nt": (_I, [_P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _P]),
    "vx_gemm_bf16_nt_variant": (_I, [_P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _I, _I, _P]),
    "vx_gemm_swiglu_bf16_nt": (_I, [_P, _P, _P, _P, _L, _L, _L, _L, _L, _L, _I, _I, _P]),
    "vx_gemm_generic": (_I, [_P, _P, _P, _P, _I] + [_L] * 13 + [_P]),
    "vx_gemm_nt_mfma": (_I, [_P, _P, _P, _P, _I, _L, _L, _L, _L, _L, _L, _P]),
    "vx_transpose_bf16": (_I, [_P, _P, _L, _L, _L, _L, _P]),
    "vx_store_kvcache": (_I, [_P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _P]),
    "vx_store_kvcache_strided": (_I, [_P, _P, _P, _P, _P, _L, _I, _L, _L, _L, _L, _I, _L, _L, _L, _L, _L, _L, _P]),
    "vx_attn_chunk_size": (_I, []),
    "vx_paged_attn_decode_workspace_bytes": (_L, [_L, _L, _L, _L, _L]),
    "vx_paged_attn_decode_workspace_needed": (_L, [_L, _L, _L, _L, _L, _I]),
    "vx_attention": (
        _I,
        [_P] * 8 + [_L, _L, _I, _I, _I, _I] + [_L] * 12 + [_I, _F, _I, _I, _I, _P, _L, _P],
    ),
    "vx_attention_ex": (
        _I,
        [_P] * 10 + [_L, _L, _I, _I, _I, _I] + [_L] * 12 + [_I, _F, _I, _I, _I, _P, _L, _P],
    ),
    "vx_attention_typed": (
        _I,
        [_P] * 10 + [_L, _L, _I, _I, _I, _I] + [_L] * 12 + [_I, _F, _I, _I, _I, _I, _P, _L, _P],
    ),
    "vx_attention_bwd_workspace_bytes": (_L, [_L, _L]),
    "vx_attention_bwd": (_I, [_P] * 11 + [_L, _L, _L, _I, _I, _I, _P, _F, _I, _I, _P, _L, _P]),
    "vx_attention_bwd_typed": (_I, [_P] * 11 + [_L, _L, _L, _I, _I, _I, _I, _P, _F, _I, _I, _I, _P, _L, _P]),
    "vx_router_topk": (_I, [_P, _P, _P, _L, _I, _I, _L, _I, _I, _I, _I, _P]),
    "vx_moe_max_tiles": (_L, [_L, _I, _I]),
    "vx_moe_route": (_I, [_P, _I, _L, _I, _I, _I] + [_P] * 8 + [_L, _P]),
    "vx_moe_route_workspace_bytes": (_L, [_L, _I]),
    "vx_moe_route_ws": (_I, [_P, _I, _L, _I, _I, _I] + [_P] * 8 + [_L, _P, _L, _P]),
    "vx_moe_gemm": (
        _I,
        [_P, _L, _P, _P, _L, _L, _P, _L, _L, _L, _P, _P, _P, _L, _I, _P, _P, _P, _I, _L, _P],
    ),
    "vx_packed_kchunks": (_I, [_L]),
    "vx_pack_weights": (_I, [_P, _L, _L, _L, _L, _L, _P, _P]),
    "vx_moe_gemm_packed": (_I, [_P, _L, _P, _P, _L, _P, _L, _L, _L, _P, _P, _P, _L, _I, _P, _P, _P, _I, _L, _P]),
    "vx_moe_gemm_nn": (_I, [_P, _L, _P, _P, _L, _L, _L, _P, _L, _P, _L, _L, _L, _P, _L, _L, _P, _P, _P, _L, _I, _L, _P]),
    "vx_rms_norm_bwd_workspace_bytes": (_L, [_L, _L]),
    "vx_rms_norm_bwd": (_I, [_P, _P, _P, _P, _P, _I, _L, _L, _L, _L, _L, _F, _I, _P, _L, _P]),
    "vx_logprobs_bwd": (_I, [_P, _P, _P, _P, _P, _I, _L, _L, _L, _L, _P]),
    "vx_router_topk_bwd": (_I, [_P, _P, _P, _P, _L, _I, _I, _L, _L, _I, _I, _I, _P]),
    "vx_moe_swiglu_bwd": (_I, [_P, _P, _P, _L, _L, _L, _P, _P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _P]),
    "vx_moe_gemm_tn": (_I, [_P, _L, _P, _P, _L, _P, _P, _L, _L, _L, _L, _P, _L, _L, _L, _P]),
    "vx_expert_histogram": (_I, [_P, _I, _L, _I, _P, _P]),
    "vx_moe_scatter": (_I, [_P, _P, _P, _L, _I, _L, _L, _L, _P]),
    "vx_moe_gather": (_I, [_P, _P, _P, _P, _L, _I, _L, _L, _L, _L, _P]),
    "vx_moe_gather_norm": (_I, [_P, _P, _P, _P, _L, _I, _L, _L, _L, _L, _P, _P, _L, _F, _I, _P]),
    "vx_moe_gather_norm_prefetch": (_I, [_P, _P, _P, _P, _L, _I, _L, _L, _L, _L, _P, _P, _L, _F, _I, _P, _L, _P]),
    "vx_qk_norm_rope_store": (
        _I,
        [_P, _L, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _L, _I, _I, _I, _F, _L, _I, _L, _L, _L, _P],
    ),
    "vx_rope": (_I, [_P, _P, _P, _P, _L, _I, _I, _L, _L, _L, _L, _L, _P]),
    "vx_embedding": (_I, [_P, _P, _I, _P, _L, _L, _L, _P]),
    "vx_fill_i32": (_I, [_P, _I, _L, _P]),
    "vx_sample_tokens": (_I, [_P, _I, _L, _L, _L, _F, _I, _F, _P, _P, _P, _P]),
    "vx_host_step_metadata": (_I, [_L, _P, _P, _P, _P, _I, _L, _L, _L] + [_P] * 8),
    "vx_kv_allocator_create": (_P, [_L]),
    "vx_kv_allocator_destroy": (None, [_P]),
    "vx_kv_allocator_num_free": (_L, [_P]),
    "vx_kv_allocator_allocate": (_L, [_P, _L, _L, _I, _P, _L]),
    "vx_kv_allocator_free": (_L, [_P, _P, _L]),
}

_lib = None
_lock = threading.Lock()


class VexactHipError(RuntimeError):
    pass


def lib_path() -> str:
    return LIB_PATH


def load() -> ctypes.CDLL:
    """Load the shared library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise VexactHipError(
                f"{LIB_PATH} is missing: build it with `python -m vexact_amd._build` "
                "(there is no CPU or PyTorch fallback for these ops)"
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().vx_status_string(rc).decode()
        raise VexactHipError(f"{what}: {msg} (status {rc})")
