"""Builds libt5attn.so (hand-written HIP for gfx950) in-tree with hipcc.

    python -m turbot5_amd.build            # or: from turbot5_amd.build import build; build()
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "build")
LIB = os.path.join(HERE, "libt5attn.so")

ARCH = "gfx950"
# packed fp32 VALU ops are switched off for device code on purpose
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Wno-unused-value",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

UNITS = [
    ("api.o", "api.hip", []),
    ("splitk.o", "splitk.hip", []),
    ("rmsnorm.o", "rmsnorm.hip", []),
    ("plan.o", "plan.hip", []),
    ("lut.o", "lut.hip", []),
    ("attn_bwd.o", "attn_bwd.hip", []),
    ("attn_fwd_bf16.o", "attn_fwd.hip", ["-DT5A_UNIT_DTYPE=0"]),
    ("attn_fwd_f32.o", "attn_fwd.hip", ["-DT5A_UNIT_DTYPE=1"]),
    ("attn_fwd_f16.o", "attn_fwd.hip", ["-DT5A_UNIT_DTYPE=2"]),
]


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    raise RuntimeError("hipcc not found")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"command failed ({r.returncode}): {' '.join(cmd)}\n{out}")
    if verbose and out.strip():
        print(out, flush=True)


TRACE_LIB = os.path.join(HERE, "libt5attn_trace.so")


def build(verbose: bool = False, jobs: int = 8, extra_flags=(), trace: bool = False) -> str:
    """Compile every translation unit and link the shared library; returns its path.

    ``trace``: a second library, libt5attn_trace.so, whose bf16 attention kernels stamp the shader clock at a few
    points of every work item (``bench.py --timeline`` reads them); the shipped library carries none of that."""
    obj_dir = os.path.join(OBJ, "trace") if trace else OBJ
    os.makedirs(obj_dir, exist_ok=True)
    hipcc = _hipcc()
    flags = [*FLAGS, *extra_flags] + (["-DT5A_TRACE"] if trace else [])
    cmds = []
    for obj, src, defs in UNITS:
        cmds.append([hipcc, *flags, *defs, "-c", os.path.join(CSRC, src), "-o", os.path.join(obj_dir, obj)])
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda c: _run(c, verbose), cmds))
    objs = [os.path.join(obj_dir, o) for o, _, _ in UNITS]
    lib = TRACE_LIB if trace else LIB
    _run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", lib, *objs], verbose)
    return lib


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, trace="--trace" in sys.argv))
