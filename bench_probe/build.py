"""Builds ``libodl_probe.so`` from probe.hip: the register-only MFMA loops that bench.py uses to read what the
matrix pipe delivers, and at what clock and board power, with no memory traffic at all.  A measurement aid of the
benchmark: it is not part of the FP8 library and nothing in the package loads it.

Run as ``python bench_probe/build.py`` (``__graft_entry__.build()`` does)."""

from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PROBE_LIB_PATH = os.path.join(HERE, "libodl_probe.so")


def build_probe(verbose: bool = False) -> str:
    from optimus_dl_amd.build import HIPCC_FLAGS, hipcc_path

    cmd = [hipcc_path(), *HIPCC_FLAGS, "-shared", os.path.join(HERE, "probe.hip"), "-o", PROBE_LIB_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on probe.hip:\n{r.stdout}")
    os.replace(PROBE_LIB_PATH + ".tmp", PROBE_LIB_PATH)
    return PROBE_LIB_PATH


if __name__ == "__main__":
    print(build_probe(verbose="-v" in sys.argv))
