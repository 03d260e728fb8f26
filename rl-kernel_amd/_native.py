"""ctypes binding of librlk_hip.so.  There is no fallback: a missing library is an error."""

from __future__ import annotations

import ctypes
import functools
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "librlk_hip.so")

DTYPE_BF16, DTYPE_F16, DTYPE_F32, DTYPE_F64 = 0, 1, 2, 3

_c = ctypes
_vp, _i32, _i64, _sz, _f32 = _c.c_void_p, _c.c_int32, _c.c_int64, _c.c_size_t, _c.c_float

# name -> (restype, argtypes); mirrors include/rlk_hip.h one to one
SIGNATURES = {
    "rlk_version": (_c.c_int, []),
    "rlk_device_info": (_c.c_int, [_i32, _vp, _vp]),
    "rlk_last_error": (_c.c_char_p, []),
    "rlk_linear_logp_fwd_workspace_bytes": (_c.c_int, [_i64, _i32, _i64, _i32, _c.POINTER(_sz)]),
    "rlk_linear_logp_fwd": (_c.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i64, _i32, _i64,
                                       _i64, _i32, _f32, _i64, _i32, _i32, _vp, _vp]),
    "rlk_linear_logp_fwd_static": (_c.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i64, _i64,
                                              _i32, _f32, _i64, _i32, _i32, _vp, _vp]),
    "rlk_linear_logp_fwd_pair_workspace_bytes": (_c.c_int, [_i64, _i32, _i64, _i32,
                                                            _c.POINTER(_sz)]),
    "rlk_linear_logp_fwd_pair": (_c.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz,
                                            _i64, _i32, _i64, _i64, _i32, _f32, _i64, _i32, _i32, _vp,
                                            _vp]),
    "rlk_linear_logp_bwd_workspace_bytes": (_c.c_int, [_i64, _i32, _i64, _i32, _sz,
                                                       _c.POINTER(_sz)]),
    "rlk_linear_logp_fwd_plan": (_c.c_int, [_i64, _i32, _i64, _i32, _c.POINTER(_i64)]),
    "rlk_linear_logp_bwd_plan": (_c.c_int, [_i64, _i32, _i64, _i32, _sz, _c.POINTER(_i64)]),
    "rlk_linear_logp_bwd": (_c.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz,
                                       _i64, _i32, _i64, _i64, _i32, _f32, _i64, _i32, _vp]),
    "rlk_linear_logp_bwd_accum": (_c.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz,
                                             _i64, _i32, _i64, _i64, _i32, _f32, _i64, _i32, _i32, _vp]),
    "rlk_rmsnorm_fwd": (_c.c_int, [_vp, _vp, _f32, _vp, _vp, _i64, _i32, _i32, _vp]),
    "rlk_rmsnorm_bwd_workspace_bytes": (_c.c_int, [_i64, _i32, _c.POINTER(_sz)]),
    "rlk_rmsnorm_bwd": (_c.c_int, [_vp, _vp, _f32, _vp, _vp, _vp, _vp, _sz, _i64, _i32, _i32, _vp]),
    "rlk_linear_logp_rmsnorm_fwd_workspace_bytes": (_c.c_int, [_i64, _i32, _i64, _i32,
                                                               _c.POINTER(_sz)]),
    "rlk_linear_logp_rmsnorm_fwd": (_c.c_int, [_vp, _vp, _f32, _vp, _vp, _vp, _vp, _vp, _vp, _sz,
                                               _i64, _i32, _i64, _i64, _i32, _f32, _i64, _i32, _i32,
                                               _vp, _vp]),
    "rlk_linear_logp_rmsnorm_bwd_workspace_bytes": (_c.c_int, [_i64, _i32, _i64, _i32, _sz,
                                                               _c.POINTER(_sz)]),
    "rlk_linear_logp_rmsnorm_bwd": (_c.c_int, [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                               _vp, _vp, _sz, _sz, _i64, _i32, _i64, _i64, _i32, _f32,
                                               _i64, _i32, _vp]),
    "rlk_logp_from_logits": (_c.c_int, [_vp, _i32, _vp, _vp, _i32, _vp, _vp, _i64, _i64, _i64, _vp]),
    "rlk_logp_from_logits_pair": (_c.c_int, [_vp, _vp, _i32, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _i64,
                                             _i64, _i64, _vp]),
    "rlk_logp_from_logits_bwd": (_c.c_int, [_vp, _i32, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "rlk_grpo_loss_workspace_bytes": (_c.c_int, [_i64, _c.POINTER(_sz)]),
    "rlk_grpo_loss_from_logp": (_c.c_int, [_vp, _vp, _vp, _vp, _i32, _vp, _i64, _i64, _f32, _f32,
                                           _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "rlk_linear_logp_fwd_grpo_workspace_bytes": (_c.c_int, [_i64, _i32, _i64, _i32,
                                                            _c.POINTER(_sz)]),
    "rlk_linear_logp_fwd_grpo": (_c.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i64, _i32, _i64,
                                            _i64, _i32, _f32, _i64, _i32, _i32, _vp,
                                            _vp, _vp, _vp, _i32, _vp, _i64, _f32, _f32, _vp, _vp,
                                            _vp, _vp, _vp, _vp]),
    "rlk_ratio_kl_from_logp": (_c.c_int, [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp]),
    "rlk_ratio_kl_from_logp_bwd": (_c.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp]),
    "rlk_group_advantages": (_c.c_int, [_vp, _vp, _i64, _f32, _vp, _vp]),
}

_lib = None


class NativeLibraryError(RuntimeError):
    pass


def load():
    """Load librlk_hip.so once and attach the prototypes. Raises if it was not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NativeLibraryError(
            f"{LIB_PATH} is missing: build it with `python rl-kernel_amd/build.py` "
            "(hipcc, gfx950). This package has no CPU or PyTorch fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name, None)
        if fn is None:
            raise NativeLibraryError(f"{LIB_PATH} does not export {name}; rebuild it")
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def available() -> bool:
    try:
        load()
        return True
    except (NativeLibraryError, OSError):
        return False


def check(rc: int, what: str) -> None:
    if rc == 0:
        return
    msg = load().rlk_last_error().decode()
    if rc == -1:
        raise ValueError(f"{what}: {msg}")
    if rc == -2:
        raise NotImplementedError(f"{what}: {msg}")
    raise RuntimeError(f"{what}: {msg} (code {rc})")


def on_tensor_device(fn):
    """Run ``fn`` with the GPU of its first CUDA tensor argument as the current device: the C ABI
    launches on a stream handle and HIP requires that stream's device to be current, which is not
    a given on a host with several GPUs."""

    @functools.wraps(fn)
    def guarded(*args, **kwargs):
        import torch

        for a in args:
            if isinstance(a, torch.Tensor) and a.is_cuda:
                with torch.cuda.device(a.device):
                    return fn(*args, **kwargs)
        return fn(*args, **kwargs)

    return guarded
