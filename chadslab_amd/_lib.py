"""ctypes binding of libchadq.so (the C ABI declared in include/chadq.h).

The library is the only compute path: if it is missing or fails to load, importing an operator raises.
There is no CPU or PyTorch fallback.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

import os

# CHADQ_LIB names another build of the library to load instead of the in-tree one (comparing two builds on one box)
LIB_PATH = Path(os.environ.get("CHADQ_LIB") or (Path(__file__).resolve().parent / "libchadq.so"))

# name -> (restype, argtypes); mirrors include/chadq.h one to one
SIGNATURES = {
    "chadq_version": (c_int, []),
    "chadq_last_error": (c_char_p, []),
    "chadq_arch": (c_char_p, []),
    "chadq_unpack_i4": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "chadq_pack_i4": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "chadq_dequant_i4g32": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "chadq_dequant_i8row": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "chadq_gemv_i4g32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "chadq_gemv_i4g32_splitk": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "chadq_gemv_i4g32_splitk_geglu": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "chadq_gemv_i4g32_addnorm": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                         c_int, c_void_p]),
    "chadq_gemv_i4g32_addnorm_geglu": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                         c_int, c_void_p]),
    "chadq_gemv_i8row": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "chadq_gemv_i8row_fp32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "chadq_gemm_i4g32_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "chadq_gemm_i8row_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "chadq_moe_route": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "chadq_moe_ffn_i4g32_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "chadq_moe_ffn_i4g32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_void_p, c_size_t, c_void_p]),
    "chadq_moe_ffn_i4g32_tiled": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                          c_void_p, c_size_t, c_void_p]),
    "chadq_repack_i4g32_tiles": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "chadq_unrepack_i4g32_tiles": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "chadq_embed_i4g32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "chadq_add_rmsnorm_bf16": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_float, c_void_p]),
    "chadq_rope_kv_write": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float,
                                    c_void_p]),
    "chadq_attn_decode_mqa_workspace_floats": (c_size_t, [c_int, c_int, c_int]),
    "chadq_attn_decode_mqa": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "chadq_rope_table": (c_int, [c_void_p, c_int, c_int, c_float, c_void_p]),
    "chadq_attn_decode_mqa_fused_workspace_floats": (c_size_t, [c_int, c_int, c_int]),
    "chadq_attn_decode_mqa_fused": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                            c_void_p]),
    "chadq_attn_decode_mqa_fused_oproj_i4g32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                        c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "chadq_attn_decode_mqa_fused_static": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                                   c_void_p]),
    "chadq_geglu_bf16": (c_int, [c_void_p, c_void_p, c_int, c_void_p]),
    "chadq_argmax_f32": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "chadq_gemv_i4g32_argmax_scratch_bytes": (c_size_t, [c_int, c_int]),
    "chadq_gemv_i4g32_argmax": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                        c_void_p, c_void_p]),
    "chadq_sample_topk_f32": (c_int, [c_void_p, c_int, c_int, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
}


class MoeExpertI4G32(ctypes.Structure):
    """Mirror of chadq_moe_expert_i4g32: six device pointers."""
    _fields_ = [(n, c_void_p) for n in ("wg", "sg", "wu", "su", "wd", "sd")]

_STATUS_EXC = {-1: ValueError, -2: ValueError, -3: ValueError, -4: ValueError, -5: RuntimeError, -6: RuntimeError}

_lib = None


class ChadqError(RuntimeError):
    pass


def open_library(path) -> ctypes.CDLL:
    """A build of the library at `path` with the signatures attached (load() for the in-tree one; bench.py also opens
    the measurement builds of chadslab_amd.build.build_ablations this way)."""
    lib = ctypes.CDLL(str(path))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    return lib


def load() -> ctypes.CDLL:
    """Loads libchadq.so once and attaches the signatures; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ChadqError(
            "%s not found: build it with `python -m chadslab_amd.build` (there is no fallback path)" % LIB_PATH
        )
    _lib = open_library(LIB_PATH)
    return _lib


def check(rc: int, what: str) -> None:
    """Turns a negative status into a Python exception carrying the library's message."""
    if rc == 0:
        return
    msg = load().chadq_last_error().decode("utf-8", "replace")
    raise _STATUS_EXC.get(rc, RuntimeError)("%s failed (%d): %s" % (what, rc, msg))
