"""Compiles the HIP sources under csrc/ into one C-ABI shared library for gfx950.

Run as ``python -m optimus_dl_amd.build`` (or call :func:`build`).  The library
lands beside this file as ``libodl_fp8.so``; it is built in-tree so that it
travels with the source tree to machines that have a GPU but no compiler step.
"""

from __future__ import annotations

import glob
import os
import re
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libodl_fp8.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["api.hip", "quant.hip", "gemm_fp8.hip", "gemm_tiled.hip", "gemm_pipe.hip", "gemm_stream.hip", "fused.hip", "mx.hip"]

# Per-source additions.  The compiler-scheduled tiled GEMMs: left to its own choice the compiler computes in vector
# registers but parks the accumulators in the accumulation registers between K steps, 64 copies out and 64 back per
# step of the 128 x 128 kernels (as many cycles of issue as the step's MFMAs).  Told to use the vector-register form of
# the MFMA it keeps them where they are: 220 -> 169 registers and 8-12 % off those kernels (8192 x 1024 x 2048: 22.3 ->
# 19.3 us).  The hand-scheduled kernels (gemm_stream.hip, gemm_pipe.hip) place their accumulators themselves.
EXTRA_FLAGS = {
    "gemm_tiled.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "mx.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}

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


_SGPR_OPERAND = re.compile(r"\bs(?:\[(\d+):(\d+)\]|(\d+))")
_VALU_WRITES_SGPR = re.compile(r"^(v_readlane_b32|v_readfirstlane_b32|v_cmp\w*)\s+s(?:\[(\d+):(\d+)\]|(\d+))")


def check_asm_hazards(asm_text: str, name: str = "") -> list[str]:
    """Finds vector-memory instructions written as inline asm that read a scalar register less
    than 5 wait states after a vector instruction wrote it.

    The hardware needs those wait states and the compiler inserts them for its own
    instructions, but it does not look inside asm statements.  Which registers feed an asm
    statement depends on register allocation (spilled scalars come back through
    ``v_readlane_b32``), so the generated code is checked after every build.
    """
    lines = asm_text.split("\n")
    problems = []
    in_asm = False
    for i, raw in enumerate(lines):
        text = raw.strip()
        if text.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if text.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not in_asm or not text.startswith(("buffer_", "global_", "flat_", "scratch_")):
            continue
        used = set()
        for lo, hi, one in _SGPR_OPERAND.findall(text):
            used |= set(range(int(lo), int(hi) + 1)) if lo else {int(one)}
        waited, j = 0, i - 1
        while j >= 0 and waited < 5:
            prev = lines[j].strip()
            j -= 1
            if not prev or prev.startswith((";", ".")) or prev.endswith(":"):
                continue
            nop = re.match(r"s_nop (\d+)", prev)
            if nop:
                waited += int(nop.group(1)) + 1
                continue
            w = _VALU_WRITES_SGPR.match(prev)
            if w:
                written = set(range(int(w.group(2)), int(w.group(3)) + 1)) if w.group(2) else {int(w.group(4))}
                if written & used:
                    problems.append(f"{name}:{i + 1}: '{text}' reads a scalar register {waited} wait states after '{prev}'")
            waited += 1
    return problems


def check_saturating_conversions(asm_text: str, name: str = "") -> list[str]:
    """The block-scaled casts rely on the scaled FP8 conversions of gfx950 saturating, which they do only while the
    wave's MODE.FP16_OVFL bit is set; the kernels set it first thing.  Nothing ties the conversions to that
    ``s_setreg`` in the compiler's eyes, so the order is checked in the generated code: inside every function, no
    ``v_cvt_scalef32_pk_*`` before the mode has been set."""
    problems = []
    func, mode_set = "", False
    for i, raw in enumerate(asm_text.split("\n")):
        text = raw.strip()
        m = re.match(r"^(_Z\w+):", raw)
        if m:
            func, mode_set = m.group(1), False
            continue
        if text.startswith("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 1"):
            mode_set = True
        elif text.startswith("v_cvt_scalef32_pk_") and not mode_set:
            problems.append(f"{name}:{i + 1}: '{text}' in {func} before MODE.FP16_OVFL is set")
            mode_set = True          # one report per function
    return problems


def build(verbose: bool = False, keep_asm: bool = False) -> str:
    """Compile every source and link ``libodl_fp8.so``.  Always recompiles."""
    hipcc = hipcc_path()
    objdir = os.path.join(HERE, "csrc", "_obj")
    os.makedirs(objdir, exist_ok=True)
    for stale in glob.glob(os.path.join(objdir, "*.s")):
        os.remove(stale)
    procs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        cmd += ["-save-temps=obj"]              # keeps the device assembly for the hazard check below
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
    problems = []
    for asm in sorted(glob.glob(os.path.join(objdir, "*gfx950*.s"))):
        with open(asm) as fh:
            text = fh.read()
        problems += check_asm_hazards(text, os.path.basename(asm))
        problems += check_saturating_conversions(text, os.path.basename(asm))
    if problems:
        raise RuntimeError("hazards in the generated code:\n" + "\n".join(problems))
    if not keep_asm:
        for tmpf in glob.glob(os.path.join(objdir, "*")):
            if not tmpf.endswith(".o"):
                os.remove(tmpf)
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
