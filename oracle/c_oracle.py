"""ctypes binding of oracle/rlk_oracle.c (double-precision brute force).

TEST INFRASTRUCTURE ONLY.  ``build()`` compiles the shared object with gcc;
``load()`` returns numpy-level callables.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "librlk_oracle.so")


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "rlk_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])
    return _SO


_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a, ty):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ty))


def _f64(a):
    return None if a is None else np.ascontiguousarray(np.asarray(a, dtype=np.float64))


def linear_logp(hidden, weight, targets, bias=None, temperature=1.0, ignore_index=None):
    lib = _load()
    hidden, weight, bias = _f64(hidden), _f64(weight), _f64(bias)
    t = np.ascontiguousarray(np.asarray(targets, dtype=np.int64))
    n, h = hidden.shape
    v = weight.shape[0]
    logp = np.empty(n)
    lse = np.empty(n)
    rc = lib.rlk_oracle_linear_logp_f64(
        _p(hidden, ctypes.c_double), _p(weight, ctypes.c_double), _p(bias, ctypes.c_double),
        _p(t, ctypes.c_int64), ctypes.c_int64(n), ctypes.c_int64(h), ctypes.c_int64(v),
        ctypes.c_double(temperature), ctypes.c_int64(0 if ignore_index is None else ignore_index),
        ctypes.c_int(ignore_index is not None), _p(logp, ctypes.c_double), _p(lse, ctypes.c_double))
    if rc:
        raise ValueError(f"rlk_oracle_linear_logp_f64 failed with code {rc}")
    return logp, lse


def linear_logp_backward(grad, hidden, weight, targets, bias=None, temperature=1.0,
                         ignore_index=None):
    lib = _load()
    grad, hidden, weight, bias = _f64(grad), _f64(hidden), _f64(weight), _f64(bias)
    t = np.ascontiguousarray(np.asarray(targets, dtype=np.int64))
    n, h = hidden.shape
    v = weight.shape[0]
    dh = np.empty((n, h))
    dw = np.empty((v, h))
    db = np.empty(v) if bias is not None else None
    rc = lib.rlk_oracle_linear_logp_bwd_f64(
        _p(grad, ctypes.c_double), _p(hidden, ctypes.c_double), _p(weight, ctypes.c_double),
        _p(bias, ctypes.c_double), _p(t, ctypes.c_int64), ctypes.c_int64(n), ctypes.c_int64(h),
        ctypes.c_int64(v), ctypes.c_double(temperature),
        ctypes.c_int64(0 if ignore_index is None else ignore_index),
        ctypes.c_int(ignore_index is not None), _p(dh, ctypes.c_double), _p(dw, ctypes.c_double),
        _p(db, ctypes.c_double))
    if rc:
        raise ValueError(f"rlk_oracle_linear_logp_bwd_f64 failed with code {rc}")
    return dh, dw, db


def logp_from_logits(logits, ids):
    lib = _load()
    logits = _f64(logits)
    t = np.ascontiguousarray(np.asarray(ids, dtype=np.int64))
    n, v = logits.shape
    out = np.empty(n)
    lib.rlk_oracle_logp_from_logits_f64(_p(logits, ctypes.c_double), _p(t, ctypes.c_int64),
                                        ctypes.c_int64(n), ctypes.c_int64(v),
                                        _p(out, ctypes.c_double))
    return out


def group_advantages(rewards, bounds, eps=1e-6):
    lib = _load()
    rewards = _f64(rewards)
    b = np.ascontiguousarray(np.asarray(bounds, dtype=np.int64))
    adv = np.empty_like(rewards)
    lib.rlk_oracle_group_advantages_f64(_p(rewards, ctypes.c_double), _p(b, ctypes.c_int64),
                                        ctypes.c_int64(len(b) - 1), ctypes.c_double(eps),
                                        _p(adv, ctypes.c_double))
    return adv


def grpo_from_logp(cur, old, ref, adv_tok, mask, clip_eps=0.2, beta=0.0):
    lib = _load()
    cur, old, ref, adv_tok = (_f64(np.ravel(x)) for x in (cur, old, ref, adv_tok))
    m = np.ascontiguousarray(np.ravel(np.asarray(mask)).astype(np.uint8))
    out3 = np.empty(3)
    dcur = np.empty_like(cur)
    lib.rlk_oracle_grpo_from_logp_f64(
        _p(cur, ctypes.c_double), _p(old, ctypes.c_double), _p(ref, ctypes.c_double),
        _p(adv_tok, ctypes.c_double), _p(m, ctypes.c_uint8), ctypes.c_int64(cur.size),
        ctypes.c_double(clip_eps), ctypes.c_double(beta), _p(out3, ctypes.c_double),
        _p(dcur, ctypes.c_double))
    return out3, dcur
