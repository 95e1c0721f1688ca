"""Builds chadslab_amd/libchadq.so from csrc/*.hip with hipcc for gfx950 (cross-compiles without a GPU).

Run as `python -m chadslab_amd.build` or through __graft_entry__.build().  The library is kept in-tree,
next to this file; nothing is installed.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = PKG / "csrc" / "_obj"
LIB = PKG / "libchadq.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops: keep the compiler from forming packed fp32 arithmetic (v_pk_*_f32)
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first 16 dwords of a kernel's arguments arrive in scalar registers with the wave instead of being fetched
    # by its first instructions: these kernels last 3-10 us and every one of them starts by waiting for that fetch
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


def _run(cmd):
    p = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature and says so on every file: drop that line
    err = "\n".join(l for l in p.stderr.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(map(str, cmd)), p.stdout, err))
    if err.strip():
        sys.stderr.write(err + "\n")


def build(verbose: bool = True, save_temps: bool = False) -> Path:
    srcs = sorted(CSRC.glob("*.hip"))
    if not srcs:
        raise RuntimeError("no HIP sources under %s" % CSRC)
    OBJ.mkdir(exist_ok=True)
    objs = [OBJ / (s.stem + ".o") for s in srcs]

    def one(pair):
        s, o = pair
        cmd = [HIPCC, *FLAGS, "-c", str(s), "-o", str(o)]
        if save_temps:
            cmd += ["-save-temps=obj"]
        _run(cmd)
        return o

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        list(ex.map(one, zip(srcs, objs)))
    tmp = LIB.with_suffix(".so.tmp")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)])
    os.replace(tmp, LIB)
    if verbose:
        print("built %s (%d sources)" % (LIB, len(srcs)))
    build_ablations(verbose)  # always together: the measurement builds share every other object and the whole C ABI
    return LIB


# Measurement builds (bench.py --extras moe_ablation / gemm_ablation): the same library with a part of one kernel's loop
# compiled out, so that the part's share of the time can be measured on its own.  Their results are wrong by
# construction; nothing but the bench loads them.  name -> (source file, macro definition)
ABLATIONS = {"stream": ("gemm_expert_i4g32.hip", "-DCHADQ_EXPERT_ABLATE=1"),   # expert GEMM: memory traffic without arithmetic
             "arith": ("gemm_expert_i4g32.hip", "-DCHADQ_EXPERT_ABLATE=2"),    # expert GEMM: arithmetic without weight loads
             "nodequant": ("gemm_q_bf16.hip", "-DCHADQ_GEMM_ABLATE=1")}        # prefill GEMM (128 x 64 tile): no dequantisation


def ablation_path(name: str) -> Path:
    return PKG / ("libchadq_ablate_%s.so" % name)


def build_ablations(verbose: bool = True) -> None:
    """Only the one source file of each ablation is recompiled; the other objects are those of the library."""
    def one(item):
        name, (fname, define) = item
        src = CSRC / fname
        obj = OBJ / ("ablate_%s.o" % name)
        _run([HIPCC, *FLAGS, define, "-c", str(src), "-o", str(obj)])
        return name, src, obj

    with ThreadPoolExecutor(max_workers=len(ABLATIONS)) as ex:
        done = list(ex.map(one, ABLATIONS.items()))
    for name, src, obj in done:
        others = [o for o in sorted(OBJ.glob("*.o")) if o.stem != src.stem and not o.stem.startswith("ablate_") and
                  (CSRC / (o.stem + ".hip")).exists()]
        tmp = ablation_path(name).with_suffix(".so.tmp")
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, others), str(obj)])
        os.replace(tmp, ablation_path(name))
        if verbose:
            print("built %s" % ablation_path(name))


if __name__ == "__main__":
    build(save_temps="--save-temps" in sys.argv)
