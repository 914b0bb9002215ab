"""Build recipe of libscn_hip.so (hipcc, gfx950 only).  Run: python -m lidar_ai_solution_amd.build"""
from __future__ import annotations

import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libscn_hip.so")

# -ffp-contract=off: the int8 epilogue is specified as separate fp32 multiply and add.
# -packed-fp32-ops is switched off for device code (packed fp32 instructions are not used).
# -no-hip-rt: no DT_NEEDED on a particular libamdhip64; the library binds to the HIP runtime that is
# already loaded in the process (PyTorch ships its own copy, and streams / pointers must come from
# one runtime).  capi.py preloads it; a C++ application links -lamdhip64 itself.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-fPIC", "-shared", "-fvisibility=hidden",
         "-no-hip-rt",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]


def sources():
    src = sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")) + glob.glob(os.path.join(HERE, "csrc", "*.cpp")))
    return src


def build(verbose: bool = False) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = ["hipcc", *FLAGS, "-I" + os.path.join(ROOT, "include"), *sources(), "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
