"""Compiles the HIP library in-tree: ``python -m pylo_amd.build``.

One translation unit, one ``hipcc`` line, gfx950 only.  ``-ffp-contract=off`` keeps the
accumulator updates bit-identical to the separately rounded multiply/add of the PyTorch
path (FMAs are written explicitly where they are wanted); packed-FP32 instruction
selection is disabled.
"""

import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_NAME = "libpylo_mi355.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = [os.path.join(HERE, "csrc", "pylo_mi355.hip")]
INCLUDES = [os.path.join(ROOT, "include"), os.path.join(HERE, "csrc")]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC)")


def build_library(verbose: bool = False) -> str:
    cmd = [hipcc_path(), "-O3", "--offload-arch=gfx950", "-std=c++17", "-shared", "-fPIC",
           "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
    for inc in INCLUDES:
        cmd += ["-I", inc]
    cmd += SOURCES + ["-o", LIB_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
