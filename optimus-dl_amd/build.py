"""Compiles the HIP sources under csrc/ into one C-ABI shared library for gfx950.

Run as ``python -m optimus_dl_amd.build`` (or call :func:`build`).  The library
lands beside this file as ``libodl_fp8.so``; it is built in-tree so that it
travels with the source tree to machines that have a GPU but no compiler step.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libodl_fp8.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["api.hip", "quant.hip", "gemm_fp8.hip", "gemm_tiled.hip", "gemm_pipe.hip"]

# -ffp-contract=off : the epilogues promise "multiply, round, add, round" (no FMA fusion)
# packed-fp32-ops off: never let the compiler form v_pk_*_f32 from scalar float code
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unknown-warning-option",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, /opt/rocm/bin/hipcc, PATH)")


def build(verbose: bool = False, keep_asm: bool = False) -> str:
    """Compile every source and link ``libodl_fp8.so``.  Always recompiles."""
    hipcc = hipcc_path()
    objdir = os.path.join(HERE, "csrc", "_obj")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if keep_asm:
            cmd += ["-save-temps=obj"]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    objs = []
    for src, obj, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out.strip():
            print(out)
        objs.append(obj)
    tmp = LIB_PATH + ".tmp"
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    r = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build(verbose="-v" in sys.argv, keep_asm="--asm" in sys.argv)
    print(path)
