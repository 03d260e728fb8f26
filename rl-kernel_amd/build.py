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
           "rlk_wide.hip", "rlk_rmsnorm.hip"]

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


BINDING_SRC = "rlk_torch_binding.cpp"
BINDING_NAME = "_rlk_C"
BINDING_PATH = os.path.join(LIB_DIR, BINDING_NAME + ".so")


def _binding_compile_cmd(obj: str):
    """hipcc line that compiles the PyTorch binding (host code, torch + pybind11 headers)."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce

    incs = [os.path.join(os.path.dirname(HERE), "include"), *ce.include_paths("cuda"),
            sysconfig.get_paths()["include"]]
    abi = int(bool(getattr(torch._C, "_GLIBCXX_USE_CXX11_ABI", True)))
    return [hipcc(), "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-x", "hip", "-c",
            os.path.join(CSRC, BINDING_SRC), "-o", obj, f"-DTORCH_EXTENSION_NAME={BINDING_NAME}",
            "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_API_INCLUDE_EXTENSION_H",
            f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-Wno-unused-result", *[f"-I{i}" for i in incs]]


def _binding_link_cmd(obj: str, out: str):
    from torch.utils import cpp_extension as ce

    torch_lib = ce.library_paths()[0]
    return [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", obj, "-o", out, f"-L{torch_lib}",
            "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
            f"-L{LIB_DIR}", "-lrlk_hip", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]


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
    # the compiled PyTorch binding (the reference's `_C` symbol names over this C ABI): its
    # compile runs beside the kernels', its link needs the library
    bind_obj = os.path.join(LIB_DIR, BINDING_NAME + ".o")
    bind_proc = subprocess.Popen(_binding_compile_cmd(bind_obj), stdout=subprocess.PIPE,
                                 stderr=subprocess.STDOUT)
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
    out = bind_proc.communicate()[0].decode()
    if bind_proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {BINDING_SRC}:\n{out}")
    tmp = BINDING_PATH + ".tmp"
    res = subprocess.run(_binding_link_cmd(bind_obj, tmp), stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if res.returncode != 0:
        raise RuntimeError("link of the PyTorch binding failed:\n" + res.stdout.decode())
    os.replace(tmp, BINDING_PATH)
    return LIB_PATH


if __name__ == "__main__":
    # run as a script, this directory heads sys.path and its platform.py would shadow the standard
    # library's `platform` for every later import (torch's included)
    sys.path = [p for p in sys.path if os.path.abspath(p or ".") != HERE]
    print(build(verbose="-v" in sys.argv))
