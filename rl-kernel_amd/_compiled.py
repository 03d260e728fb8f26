"""Loader of the compiled PyTorch binding ``lib/_rlk_C.so`` (pybind11, built by ``build.py`` from
``csrc/rlk_torch_binding.cpp``).  ``module()`` returns it, or ``None`` when it was not built; the
ctypes route of ``_native`` serves the same C ABI then."""

from __future__ import annotations

import importlib.util
import os

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "_rlk_C.so")
_module = None
_tried = False


def module():
    global _module, _tried
    if not _tried:
        _tried = True
        if os.path.exists(_PATH):
            spec = importlib.util.spec_from_file_location("_rlk_C", _PATH)
            mod = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(mod)
            _module = mod
    return _module
