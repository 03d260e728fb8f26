"""Builds librlk_hip.so (the C-ABI library of HIP kernels) in-tree for gfx950 with hipcc."""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "librlk_hip.so")

SOURCES = ["rlk_core.hip", "rlk_linear_logp.hip", "rlk_logp_scan.hip", "rlk_grpo.hip",
           "rlk_generic.hip"]

# Packed-fp32 VALU forms are switched off for every device function of this library.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; librlk_hip.so cannot be built")
    return exe


def build(verbose: bool = False, extra_flags=()) -> str:
    """Compile every source and link the shared library. Always recompiles."""
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            continue
        obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
        cmd = [hipcc(), *HIPCC_FLAGS, *extra_flags, "-c", path, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    for src, proc in procs:
        out = proc.communicate()[0].decode()
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose:
            kept = [l for l in out.splitlines() if "not a recognized feature" not in l]
            if kept:
                print("\n".join(kept))
    tmp = LIB_PATH + ".tmp"
    link = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    res = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout.decode())
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
