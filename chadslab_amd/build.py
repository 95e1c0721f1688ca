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
    return LIB


# Measurement builds of the tile-order expert GEMM (bench.py --extras moe_ablation): the same library with one half of
# that kernel's loop compiled out, so that each half's share of the time can be measured on its own.  Their results are
# wrong by construction; nothing but the bench loads them.
ABLATIONS = {"stream": 1,  # memory traffic without arithmetic
             "arith": 2}   # arithmetic without weight loads


def ablation_path(name: str) -> Path:
    return PKG / ("libchadq_ablate_%s.so" % name)


def build_ablations(verbose: bool = True) -> None:
    """Needs build() to have run: only gemm_expert_i4g32.hip is recompiled, the other objects are shared."""
    src = CSRC / "gemm_expert_i4g32.hip"
    others = [o for o in sorted(OBJ.glob("*.o")) if o.stem != src.stem and not o.stem.startswith("ablate_") and
              (CSRC / (o.stem + ".hip")).exists()]
    for name, mode in ABLATIONS.items():
        obj = OBJ / ("ablate_%s.o" % name)
        _run([HIPCC, *FLAGS, "-DCHADQ_EXPERT_ABLATE=%d" % mode, "-c", str(src), "-o", str(obj)])
        tmp = ablation_path(name).with_suffix(".so.tmp")
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, others), str(obj)])
        os.replace(tmp, ablation_path(name))
        if verbose:
            print("built %s" % ablation_path(name))


if __name__ == "__main__":
    build(save_temps="--save-temps" in sys.argv)
    if "--ablations" in sys.argv:
        build_ablations()
