"""Builds and loads the scalar C twin of the oracle (oracle/chadq_oracle.c -> oracle/liboracle_c.so).

TEST INFRASTRUCTURE ONLY.  There is no reference source to compile into oracle/_ref: the reference snapshot
has no implementation of this path, so the recipe below covers the restatement alone.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import POINTER, c_double, c_float, c_int, c_int8, c_int32, c_int64, c_uint8, c_uint16
from pathlib import Path

HERE = Path(__file__).resolve().parent
SRC = HERE / "chadq_oracle.c"
LIB = HERE / "liboracle_c.so"


def build(force: bool = False) -> Path:
    if force or not LIB.exists() or LIB.stat().st_mtime < SRC.stat().st_mtime:
        tmp = LIB.with_suffix(".so.tmp")
        subprocess.run(["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-Wall", "-o", str(tmp), str(SRC), "-lm"], check=True)
        os.replace(tmp, LIB)
    return LIB


def load() -> ctypes.CDLL:
    lib = ctypes.CDLL(str(build()))
    u8p, i8p, u16p, f32p, f64p, i32p = (POINTER(t) for t in (c_uint8, c_int8, c_uint16, c_float, c_double, c_int32))
    sig = {
        "oracle_bf16_to_f32": [u16p, f32p, c_int64],
        "oracle_f32_to_bf16": [f32p, u16p, c_int64],
        "oracle_f16_to_f32": [u16p, f32p, c_int64],
        "oracle_unpack_i4": [u8p, i8p, c_int64],
        "oracle_pack_i4": [i8p, u8p, c_int64],
        "oracle_gemm_i8row_f64": [f32p, i8p, f32p, f64p, c_int, c_int, c_int],
        "oracle_gemm_i4g32_f64": [u16p, u8p, u16p, f64p, c_int, c_int, c_int],
        "oracle_gemm_i4g32_f32": [u16p, u8p, u16p, f32p, c_int, c_int, c_int],
        "oracle_moe_route": [f32p, i32p, f32p, c_int, c_int, c_int, c_int],
        "oracle_silu": [f32p, f32p, c_int64],
    }
    for name, args in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = None
    return lib


def ptr(a, ctype):
    """numpy array -> ctypes pointer of the given element type (array must be C-contiguous)."""
    return a.ctypes.data_as(POINTER(ctype))


if __name__ == "__main__":
    print(build(force=True))
