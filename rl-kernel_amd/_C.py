"""Native symbol table of the gfx950 backend, under the names the reference's compiled module
exposes (csrc/ops.cpp:75-99, rl_engine/_C.pyi:5-43 of the reference) so that wrappers probing
``hasattr(_C, name)`` find them.  ``fused_linear_logp`` is the device-neutral name of what the
reference calls ``fused_linear_logp_sm90``; both names are bound.

Two routes to the same C ABI: the compiled PyTorch extension ``lib/_rlk_C.so`` (pybind11, built by
``build.py`` from ``csrc/rlk_torch_binding.cpp``) when it is there, otherwise the ctypes wrappers
below.  ``COMPILED`` says which one is bound."""

from __future__ import annotations

from typing import List, Optional

import torch

from . import _compiled
from .ops.linear_logp import _aligned_contiguous, fused_linear_logp_forward
from .ops.logp import logp_from_logits


def _check_2d(logits):
    if logits.dim() != 2:
        raise RuntimeError("logits must be a 2D tensor")


def fused_logp_forward_out(logits, token_ids, output):
    return logp_from_logits(logits, token_ids, output)


def fused_logp(logits, token_ids):
    _check_2d(logits)
    return logp_from_logits(logits, token_ids, torch.empty(logits.size(0), device=logits.device,
                                                           dtype=logits.dtype))


def fused_logp_forward_fp32(logits, token_ids):
    _check_2d(logits)
    return logp_from_logits(logits, token_ids, torch.empty(logits.size(0), device=logits.device,
                                                           dtype=torch.float32))


def fused_logp_forward_indexed_out(logits, token_ids, row_indices, output):
    return logp_from_logits(logits, token_ids, output, row_indices)


def fused_logp_forward_indexed_fp32(logits, token_ids, row_indices):
    _check_2d(logits)
    out = torch.zeros(logits.size(0), device=logits.device, dtype=torch.float32)
    return logp_from_logits(logits, token_ids, out, row_indices)


fused_logp_forward_online_out = fused_logp_forward_out
fused_logp_forward_online_fp32 = fused_logp_forward_fp32
fused_logp_forward_online_indexed_out = fused_logp_forward_indexed_out
fused_logp_forward_online_indexed_fp32 = fused_logp_forward_indexed_fp32


def fused_linear_logp(hidden: torch.Tensor, weight: torch.Tensor, target: torch.Tensor,
                      bias: Optional[torch.Tensor] = None) -> List[torch.Tensor]:
    """``[logp, lse]`` fp32 of a (possibly vocab-sharded) head; targets outside the shard give
    ``logp = -lse`` (z_t = 0), as the reference kernel does."""
    if hidden.dim() != 2 or weight.dim() != 2:
        raise RuntimeError("hidden and weight must be 2D tensors")
    if not (hidden.is_cuda and weight.is_cuda):
        raise RuntimeError("hidden and weight must be CUDA tensors")
    if weight.size(1) != hidden.size(1):
        raise RuntimeError("hidden/weight hidden-dim mismatch")
    if target.numel() != hidden.size(0):
        raise RuntimeError(f"target must have one id per token: expected {hidden.size(0)} "
                           f"(hidden rows), got {target.numel()}")
    logp, lse, _ = fused_linear_logp_forward(
        _aligned_contiguous(hidden), _aligned_contiguous(weight),
        target.reshape(-1).to(device=hidden.device, dtype=torch.long).contiguous(), bias,
        strict_targets=False)
    return [logp, lse]


fused_linear_logp_sm90 = fused_linear_logp



_PYTHON_ROUTE = {name: obj for name, obj in list(globals().items())
                 if name.startswith("fused_") and callable(obj)}
compiled_module = _compiled.module()
COMPILED = compiled_module is not None
if COMPILED:
    for _name in _PYTHON_ROUTE:
        if hasattr(compiled_module, _name):
            globals()[_name] = getattr(compiled_module, _name)
