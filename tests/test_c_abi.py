"""The C-ABI library loads without a GPU and exports exactly what include/vexact_hip.h declares."""

import ctypes
import os
import re

from vexact_amd import _build, _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "vexact_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vx_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built_and_loads():
    if not os.path.exists(_build.LIB_PATH):
        _build.build()
    lib = _lib.load()
    assert lib.vx_abi_version() == 8
    assert lib.vx_status_string(0) == b"ok"
    assert b"workspace" in lib.vx_status_string(-3)


def test_every_declared_symbol_is_exported_and_bound():
    names = _declared()
    assert len(names) >= 25
    lib = ctypes.CDLL(_build.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert sorted(_lib.PROTOTYPES) == names, "ctypes prototypes and header out of sync"


def test_host_only_helpers():
    lib = _lib.load()
    assert lib.vx_attn_chunk_size() == 256
    # partial states: (Dv + 2) floats per (sequence, head, 256-key chunk)
    # one 9-slot (8 accumulator + 1 max/sum) x 64-lane x 16-byte image per (sequence, kv head, chunk)
    assert lib.vx_paged_attn_decode_workspace_bytes(64, 16, 4, 128, 4096) == 64 * 4 * 16 * 9 * 1024
    assert lib.vx_paged_attn_decode_workspace_bytes(1, 1, 1, 128, 1) == 9 * 1024
    assert lib.vx_paged_attn_decode_workspace_bytes(2, 64, 2, 256, 257) == 2 * 2 * 2 * (2 * 2 * 8 + 2) * 1024
    # what a launch really uses: nothing when the fused decode form is taken (mode 4, or mode 0 from 512 (sequence, kv head) pairs)
    assert lib.vx_paged_attn_decode_workspace_needed(256, 32, 4, 128, 4096, 0) == 0
    assert lib.vx_paged_attn_decode_workspace_needed(64, 16, 8, 128, 4096, 0) == 0
    assert lib.vx_paged_attn_decode_workspace_needed(8, 32, 4, 128, 4096, 0) == lib.vx_paged_attn_decode_workspace_bytes(8, 32, 4, 128, 4096)
    assert lib.vx_paged_attn_decode_workspace_needed(256, 32, 4, 128, 4096, 3) == lib.vx_paged_attn_decode_workspace_bytes(256, 32, 4, 128, 4096)
    assert lib.vx_paged_attn_decode_workspace_needed(8, 32, 4, 128, 4096, 4) == 0
    assert lib.vx_paged_attn_decode_workspace_needed(8, 32, 4, 128, 4096, 1) == 0  # not a decode mode
    # 16 bytes per (row, 4096-column chunk)
    assert lib.vx_log_softmax_workspace_bytes(7, 151936) == 7 * 38 * 16
    assert lib.vx_moe_max_tiles(2048, 128, 32) == 128 + 64
    assert lib.vx_moe_max_tiles(8, 128, 32) == 8
    assert lib.vx_moe_max_tiles(0, 128, 32) == 0


def test_bad_arguments_are_rejected_before_any_launch():
    lib = _lib.load()
    assert lib.vx_gemm_bf16_nt(None, None, None, None, 1, 1, 8, 8, 8, 8, None) == -1
    assert lib.vx_rms_norm(None, None, None, None, None, 1, 1, 8, 8, 0, 8, 0, 1e-6, 0, None) == -1
    assert lib.vx_moe_route(None, 0, 1, 1, 1, 32, None, None, None, None, None, None, None, None, 8, None) == -1
    assert lib.vx_attention(None, None, None, None, None, None, None, None, 1, 1, 4, 2, 128, 128,
                            0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 16, 1.0, 1, 0, 1, None, 0, None) == -1


def _header_signatures():
    """name -> (return type, [parameter types]) parsed from the header: 'ptr' for any pointer or the stream handle,
    else the scalar type."""
    text = open(os.path.join(ROOT, "include", "vexact_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    sigs = {}
    for m in re.finditer(r"([A-Za-z_][A-Za-z0-9_ ]*?[\s\*]+)(vx_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        ret, name, params = m.group(1).strip(), m.group(2), m.group(3).strip()

        def kind(decl: str) -> str:
            decl = decl.strip()
            if "*" in decl or decl.startswith("hipStream_t"):
                return "ptr"
            return re.sub(r"\s+[A-Za-z_][A-Za-z0-9_]*$", "", re.sub(r"^const\s+", "", decl)).strip()

        plist = [] if params in ("", "void") else [kind(p) for p in params.split(",")]
        sigs[name] = (kind(ret + " x") if "*" not in ret else "ptr", plist)
    return sigs


def test_ctypes_prototypes_match_the_header_parameter_by_parameter():
    want = {"ptr": ctypes.c_void_p, "int": ctypes.c_int, "int32_t": ctypes.c_int, "int64_t": ctypes.c_int64, "float": ctypes.c_float,
            "void": None}
    sigs = _header_signatures()
    assert sorted(sigs) == sorted(_lib.PROTOTYPES)
    for name, (ret, params) in sigs.items():
        restype, argtypes = _lib.PROTOTYPES[name]
        assert len(argtypes) == len(params), f"{name}: {len(argtypes)} ctypes arguments, {len(params)} in the header"
        for i, (a, p) in enumerate(zip(argtypes, params)):
            assert a is want[p], f"{name}: argument {i} is {p} in the header, {a.__name__} in the binding"
        if ret == "ptr":
            assert restype in (ctypes.c_char_p, ctypes.c_void_p), name
        else:
            assert restype is want[ret], f"{name}: returns {ret} in the header, {restype.__name__} in the binding"


def _source_definitions():
    """name -> [parameter kinds] of every vx_* function DEFINED in csrc (the sources do not include the public header,
    so nothing else compares the two)."""
    src_dir = os.path.join(ROOT, "vexact_amd", "csrc")
    defs = {}
    for fn in sorted(os.listdir(src_dir)):
        if not fn.endswith((".hip", ".cpp")):
            continue
        text = open(os.path.join(src_dir, fn)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        for m in re.finditer(r"\b(vx_[a-z0-9_]+)\s*\(([^;{}()]*)\)\s*\{", text, flags=re.S):
            name, params = m.group(1), m.group(2).strip()

            def kind(decl: str) -> str:
                decl = decl.strip()
                if "*" in decl or decl.startswith("hipStream_t"):
                    return "ptr"
                return re.sub(r"\s+[A-Za-z_][A-Za-z0-9_]*$", "", re.sub(r"^const\s+", "", decl)).strip()

            plist = [] if params in ("", "void") else [kind(p) for p in params.split(",")]
            assert name not in defs, f"{name} defined twice ({fn})"
            defs[name] = plist
    return defs


def test_definitions_in_the_sources_match_the_header():
    sigs, defs = _header_signatures(), _source_definitions()
    assert sorted(defs) == sorted(sigs), set(defs) ^ set(sigs)
    for name, (_, params) in sigs.items():
        assert defs[name] == params, f"{name}: header {params}, definition {defs[name]}"
