"""RMSNorm on MI355X: the step in front of the fused linear log-prob.

``RocmRMSNormOp`` has the interface of the reference's ``NativeRMSNormOp``
(rl_engine/kernels/ops/pytorch/norm/rms_norm.py:9-70): ``op(x, weight, eps=1e-6)`` returns
``x * rsqrt(mean(x^2, -1) + eps) * weight`` accumulated in fp32 and cast to ``x.dtype``;
``forward_fp32`` forces an fp32 result.  Differentiable w.r.t. ``x`` and ``weight``.
"""

from __future__ import annotations

import torch

from .. import _native
from ..platform import logger
from .linear_logp import _DTYPES, _aligned_contiguous, _ptr, _stream


@_native.on_tensor_device
def rmsnorm_forward(x_2d: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """Raw launch: normalised rows in the dtype of ``x_2d`` ([N, H] contiguous, gain [H] float32)."""
    out = torch.empty_like(x_2d)
    n, h = x_2d.shape
    if n == 0:
        return out
    gain = _aligned_contiguous(gain.detach().to(torch.float32))
    rc = _native.load().rlk_rmsnorm_fwd(_ptr(x_2d), _ptr(gain), float(eps), _ptr(out), None, n, h,
                                        _DTYPES[x_2d.dtype], _stream(x_2d.device))
    _native.check(rc, "rlk_rmsnorm_fwd")
    return out


@_native.on_tensor_device
def rmsnorm_backward(x_2d: torch.Tensor, gain: torch.Tensor, eps: float, d_out: torch.Tensor):
    """Raw launch: ``(d_x [N, H] in the dtype of x, d_gain [H] fp32)``."""
    lib = _native.load()
    n, h = x_2d.shape
    d_x = torch.empty_like(x_2d)
    d_gain = torch.zeros(h, device=x_2d.device, dtype=torch.float32)
    if n == 0:
        return d_x, d_gain
    gain = _aligned_contiguous(gain.detach().to(torch.float32))
    need = _native.ctypes.c_size_t(0)
    _native.check(lib.rlk_rmsnorm_bwd_workspace_bytes(n, h, _native.ctypes.byref(need)),
                  "rmsnorm backward workspace query")
    ws = torch.empty(max(need.value, 16), device=x_2d.device, dtype=torch.uint8)
    rc = lib.rlk_rmsnorm_bwd(_ptr(x_2d), _ptr(gain), float(eps), _ptr(d_out), _ptr(d_x), _ptr(d_gain),
                             _ptr(ws), ws.numel(), n, h, _DTYPES[x_2d.dtype], _stream(x_2d.device))
    _native.check(rc, "rlk_rmsnorm_bwd")
    return d_x, d_gain


class _RMSNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        x_2d = _aligned_contiguous(x.reshape(-1, x.size(-1)))
        gain = _aligned_contiguous(weight.detach().to(torch.float32))  # the reference multiplies by weight.float()
        ctx.save_for_backward(x_2d, gain)
        ctx.eps = eps
        ctx.x_shape = x.shape
        ctx.weight_dtype = weight.dtype
        return rmsnorm_forward(x_2d, gain, eps).reshape(x.shape)

    @staticmethod
    def backward(ctx, grad_out):
        x_2d, gain = ctx.saved_tensors
        d_out = _aligned_contiguous(grad_out.reshape(x_2d.shape).to(x_2d.dtype))
        d_x, d_gain = rmsnorm_backward(x_2d, gain, ctx.eps, d_out)
        return (d_x.reshape(ctx.x_shape) if ctx.needs_input_grad[0] else None,
                d_gain.to(ctx.weight_dtype) if ctx.needs_input_grad[1] else None, None)


class RocmRMSNormOp:
    """gfx950 RMSNorm (fp32 accumulate, one cast).  Constructor raises ``RuntimeError`` when the
    HIP library or a ROCm GPU is missing."""

    def __init__(self) -> None:
        if not torch.cuda.is_available() or getattr(torch.version, "hip", None) is None:
            raise RuntimeError("RocmRMSNormOp needs a ROCm GPU")
        _native.load()
        logger.info("Linked to librlk_hip.so RMSNorm kernels.")

    def __call__(self, x: torch.Tensor, weight: torch.Tensor, *, eps: float = 1e-6) -> torch.Tensor:
        return self.forward(x, weight, eps=eps)

    @staticmethod
    def _check(x: torch.Tensor, weight: torch.Tensor) -> None:
        if weight.dim() != 1 or weight.shape[0] != x.shape[-1]:
            raise ValueError(f"weight must be 1-D of size x.shape[-1]={x.shape[-1]}, "
                             f"got tuple(weight.shape)={tuple(weight.shape)}")
        if not (x.is_cuda and weight.is_cuda and x.device == weight.device) or x.dtype not in _DTYPES:
            raise NotImplementedError("RocmRMSNormOp needs bf16 / f16 / f32 tensors on one GPU")

    def forward(self, x: torch.Tensor, weight: torch.Tensor, *, eps: float = 1e-6) -> torch.Tensor:
        """Accumulate in fp32, cast the result back to ``x.dtype``."""
        self._check(x, weight)
        return _RMSNormFunction.apply(x, weight, float(eps))

    def forward_fp32(self, x: torch.Tensor, weight: torch.Tensor, *, eps: float = 1e-6) -> torch.Tensor:
        """Accumulate in fp32 and return fp32 (the inputs are upcast, which is exact)."""
        self._check(x, weight)
        return _RMSNormFunction.apply(x.float(), weight.float(), float(eps))
