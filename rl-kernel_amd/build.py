"""Builds librlk_hip.so (the C-ABI library of HIP kernels) in-tree for gfx950 with hipcc."""

from __future__ import annotations

import os
import re
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "librlk_hip.so")

SOURCES = ["rlk_core.hip", "rlk_linear_logp.hip", "rlk_logp_scan.hip", "rlk_grpo.hip",
           "rlk_generic.hip", "rlk_rmsnorm.hip"]

# Packed-fp32 VALU forms are switched off for every device function of this library (the host pass
# of hipcc warns that it does not know the feature; build() checks the device code instead).
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


def _check_no_packed_fp32(asm_path: str, src: str) -> None:
    """The switch-off of the packed-fp32 VALU forms is a device-side target feature; the host pass
    of hipcc does not know it and says so.  What counts is the device code: it must not contain
    a packed fp32 add / mul / fma."""
    bad = re.compile(r"\bv_pk_(add|mul|fma)_f32\b")
    with open(asm_path) as fh:
        hits = [line.strip() for line in fh if bad.search(line)]
    if hits:
        raise RuntimeError(f"{src}: device code contains packed fp32 instructions "
                           f"({len(hits)}, first: {hits[0]}); the -packed-fp32-ops switch did not take effect")


def build(verbose: bool = False, extra_flags=()) -> str:
    """Compile every source and link the shared library. Always recompiles.  Every source is
    also compiled to device assembly once more to verify that no packed-fp32 instruction was
    generated."""
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            raise RuntimeError(f"source file {path} is missing")
        obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
        asm = os.path.join(LIB_DIR, src.replace(".hip", ".device.s"))
        cmd = [hipcc(), *HIPCC_FLAGS, *extra_flags, "-c", path, "-o", obj]
        chk = [hipcc(), *HIPCC_FLAGS, *extra_flags, "--cuda-device-only", "-S", path, "-o", asm]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, None, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        procs.append((src, asm, subprocess.Popen(chk, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        objs.append(obj)
    for src, asm, proc in procs:
        out = proc.communicate()[0].decode()
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and asm is None and out.strip():
            print(out)
        if asm is not None:
            _check_no_packed_fp32(asm, src)
            os.remove(asm)
    tmp = LIB_PATH + ".tmp"
    link = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    res = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout.decode())
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
