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


# Kernels whose memory waits are counted by hand (s_waitcnt vmcnt(N) names which load has landed): a register spill
# adds scratch loads to that counter behind the code's back, so a build in which one of them uses scratch memory fails.
# The compiler reports every kernel's resources as remarks; they are read from the output of these translation units.
NO_SCRATCH_KERNELS = ("k_conv_lds",)   # (k_conv_tile and k_conv_rows leave their waits to the compiler)
RESOURCE_REMARKS = "-Rpass-analysis=kernel-resource-usage"


def kernels_with_scratch(compiler_output: str):
    """[(mangled kernel name, bytes per lane)] of the hand-counted kernels that the remarks report scratch for."""
    found, name = [], None
    for line in compiler_output.splitlines():
        if "remark:" not in line:
            continue
        if "Function Name:" in line:
            name = line.split("Function Name:", 1)[1].split("[", 1)[0].strip()
        elif "ScratchSize [bytes/lane]:" in line and name is not None:
            size = int(line.split("ScratchSize [bytes/lane]:", 1)[1].split("[", 1)[0].strip())
            if size > 0 and any(k in name for k in NO_SCRATCH_KERNELS):
                found.append((name, size))
    return found


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    spilled = kernels_with_scratch(proc.stdout) if RESOURCE_REMARKS in cmd else []
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and "kernel-resource-usage" not in l
                    and not (RESOURCE_REMARKS in cmd and (l.lstrip().startswith(("|", "^")) or "__launch_bounds__" in l
                                                          or l.startswith("In file included"))))
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed: " + " ".join(cmd) + "\n" + out)
    if spilled:
        if "-o" in cmd and os.path.exists(cmd[cmd.index("-o") + 1]):
            os.remove(cmd[cmd.index("-o") + 1])   # (an incremental build must not pick the object up later)
        raise RuntimeError("kernels with hand-counted memory waits use scratch memory (register spills):\n" +
                           "\n".join(f"  {n}: {b} bytes per lane" for n, b in spilled))
    if verbose and out.strip():
        print(out)


def _stamp(cmd) -> str:
    """What an object file was compiled with: the command line (flags, include paths) and the list of kernels whose
    scratch use fails the build.  Kept next to the object; an object whose stamp differs is compiled again, so that
    the scratch check has run with the current rules on everything that is linked."""
    import hashlib
    return hashlib.sha256(("\0".join(cmd) + "\0" + ",".join(NO_SCRATCH_KERNELS)).encode()).hexdigest()


def _stale(obj: str, src: str, cmd) -> bool:
    """True when obj is older than its source or than any header of csrc/ and include/ (all levels), or was
    compiled with another command line."""
    if not os.path.exists(obj) or not os.path.exists(obj + ".stamp"):
        return True
    with open(obj + ".stamp") as f:
        if f.read().strip() != _stamp(cmd):
            return True
    t = os.path.getmtime(obj)
    deps = [src] + glob.glob(os.path.join(HERE, "csrc", "*.hpp")) + \
        [p for p in glob.glob(os.path.join(ROOT, "include", "**", "*"), recursive=True) if os.path.isfile(p)]
    return any(os.path.getmtime(d) > t for d in deps)


def build(verbose: bool = False, jobs: int = 0, incremental: bool = False) -> str:
    """Compiles every source to an object file (side by side, `jobs` at a time) and links the library.
    incremental: keep the object files that are newer than their source and every header."""
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    compile_flags = [f for f in FLAGS if f not in ("-shared", "-no-hip-rt")]
    jobs_ = jobs or min(8, os.cpu_count() or 1)
    objs = []
    cmds = []
    for src in sources():
        obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
        objs.append(obj)
        remarks = [RESOURCE_REMARKS] if os.path.basename(src).startswith("scn_conv_") else []
        cmd = ["hipcc", *compile_flags, *remarks, "-I" + os.path.join(ROOT, "include"), "-c", src, "-o", obj]
        if incremental and not _stale(obj, src, cmd):
            continue
        cmds.append(cmd)

    def compile_one(cmd):
        obj = cmd[cmd.index("-o") + 1]
        if os.path.exists(obj + ".stamp"):
            os.remove(obj + ".stamp")
        _run(cmd, verbose)
        with open(obj + ".stamp", "w") as f:
            f.write(_stamp(cmd))

    if cmds and os.path.exists(LIB_PATH):
        os.remove(LIB_PATH)    # (a build that fails must not leave the library of older sources behind)
    with ThreadPoolExecutor(max_workers=jobs_) as pool:
        list(pool.map(compile_one, cmds))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-fvisibility=hidden", "-no-hip-rt", *objs, "-o", LIB_PATH],
         verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True, incremental="--incremental" in sys.argv))
    sys.exit(0)
