"""Selected-token log-prob from materialised logits on MI355X (the ``fused_logp`` family).

``RocmFusedLogpOp`` has the nine-method API of the reference's ``logp`` backends
(rl_engine/kernels/ops/pytorch/loss/logp.py:7-103, rl_engine/kernels/ops/cuda/loss/logp.py:92-205;
method list pinned by tests/test_op_accuracy.py:46-57 of the reference).  Every method is one
launch of the single-pass online-softmax scan kernel; the ``online_*`` names are aliases because
the two-pass and the online formulations compute the same value.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import _native
from ..platform import logger

_IN = {torch.bfloat16: _native.DTYPE_BF16, torch.float16: _native.DTYPE_F16,
       torch.float32: _native.DTYPE_F32}
_OUT = dict(_IN)
_OUT[torch.float64] = _native.DTYPE_F64


def _stream(device):
    return torch.cuda.current_stream(device).cuda_stream


@_native.on_tensor_device
def logp_from_logits(logits_2d: torch.Tensor, ids_1d: torch.Tensor, output_1d: torch.Tensor,
                     row_indices: Optional[torch.Tensor] = None,
                     lse_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Raw launch: writes ``output_1d`` (all rows, or only ``row_indices``) and returns it."""
    lib = _native.load()
    if logits_2d.dim() != 2:
        raise RuntimeError("logits must be a 2D tensor")
    if ids_1d.dim() != 1 or output_1d.dim() != 1:
        raise RuntimeError("token_ids and output must be 1D tensors")
    if not (logits_2d.is_cuda and ids_1d.is_cuda and output_1d.is_cuda):
        raise RuntimeError("logits, token_ids and output must be CUDA tensors")
    if not (logits_2d.device == ids_1d.device == output_1d.device):
        raise RuntimeError("logits, token_ids and output must be on the same CUDA device")
    if ids_1d.dtype != torch.long:
        raise RuntimeError("token_ids must be int64")
    n, v = logits_2d.shape
    if ids_1d.numel() != n:
        raise RuntimeError("token_ids length must match logits rows")
    if output_1d.numel() != n:
        raise RuntimeError("output length must match logits rows")
    if not output_1d.is_contiguous():
        raise RuntimeError("output must be contiguous")
    if v <= 0:
        raise RuntimeError("logits vocab dimension must be non-empty")
    if logits_2d.dtype not in _IN:
        raise RuntimeError("logits dtype must be float32, float16 or bfloat16")
    if output_1d.dtype not in _OUT:
        raise RuntimeError("output dtype must be float64, float32, float16, or bfloat16")
    logits_c = logits_2d.contiguous()
    ids_c = ids_1d.contiguous()
    idx_c = None
    n_launch = n
    if row_indices is not None:
        if row_indices.dim() != 1 or row_indices.dtype != torch.long or not row_indices.is_cuda:
            raise RuntimeError("row_indices must be a 1D int64 CUDA tensor")
        idx_c = row_indices.contiguous()
        n_launch = idx_c.numel()
    rc = lib.rlk_logp_from_logits(
        logits_c.data_ptr(), _IN[logits_c.dtype], ids_c.data_ptr(), output_1d.data_ptr(),
        _OUT[output_1d.dtype], None if lse_out is None else lse_out.data_ptr(),
        None if idx_c is None else idx_c.data_ptr(), n_launch, n, v, _stream(logits_c.device))
    _native.check(rc, "rlk_logp_from_logits")
    return output_1d


class RocmFusedLogpOp:
    """HIP single-pass selected-token log-prob with the reference's RL variants.

    A token id outside ``[0, V)`` yields 0 rather than an error, as in the reference's native
    kernels (csrc/fused_logp_kernel.cu:147-155)."""

    def __init__(self) -> None:
        if not torch.cuda.is_available() or getattr(torch.version, "hip", None) is None:
            raise RuntimeError("RocmFusedLogpOp needs a ROCm GPU")
        _native.load()
        logger.info("Linked to librlk_hip.so logp scan kernel.")

    def __call__(self, logits: torch.Tensor, token_ids: torch.Tensor) -> torch.Tensor:
        return self.apply(logits, token_ids)

    # ---- helpers --------------------------------------------------------------------------
    @staticmethod
    def _prepare_inputs(logits, token_ids):
        if logits.shape[:-1] != token_ids.shape:
            raise ValueError(
                f"logits leading shape {tuple(logits.shape[:-1])} must match "
                f"token_ids shape {tuple(token_ids.shape)}")
        orig_shape = logits.shape[:-1]
        logits_2d = logits.reshape(-1, logits.size(-1))
        ids_1d = token_ids.reshape(-1).to(device=logits.device, dtype=torch.long).contiguous()
        return logits_2d, ids_1d, orig_shape

    @staticmethod
    def _prepare_output(output, orig_shape):
        if output.shape != orig_shape:
            raise ValueError(
                f"output shape {tuple(output.shape)} must match logits leading shape "
                f"{tuple(orig_shape)}")
        if not output.is_contiguous():
            raise RuntimeError("output must be contiguous")
        return output.view(-1)

    @staticmethod
    def _prepare_indices(row_indices, logits):
        return row_indices.reshape(-1).to(device=logits.device, dtype=torch.long).contiguous()

    # ---- the nine methods -----------------------------------------------------------------
    def apply(self, logits, token_ids):
        logits_2d, ids_1d, shape = self._prepare_inputs(logits, token_ids)
        out = torch.empty(logits_2d.size(0), device=logits.device, dtype=logits.dtype)
        return logp_from_logits(logits_2d, ids_1d, out).view(shape)

    def apply_fp32(self, logits, token_ids):
        logits_2d, ids_1d, shape = self._prepare_inputs(logits, token_ids)
        out = torch.empty(logits_2d.size(0), device=logits.device, dtype=torch.float32)
        return logp_from_logits(logits_2d, ids_1d, out).view(shape)

    def out(self, logits, token_ids, output):
        logits_2d, ids_1d, shape = self._prepare_inputs(logits, token_ids)
        logp_from_logits(logits_2d, ids_1d, self._prepare_output(output, shape))
        return output

    def indexed_out(self, logits, token_ids, row_indices, output):
        logits_2d, ids_1d, shape = self._prepare_inputs(logits, token_ids)
        idx = self._prepare_indices(row_indices, logits)
        logp_from_logits(logits_2d, ids_1d, self._prepare_output(output, shape), idx)
        return output

    def indexed_fp32(self, logits, token_ids, row_indices):
        output = torch.zeros(logits.shape[:-1], device=logits.device, dtype=torch.float32)
        return self.indexed_out(logits, token_ids, row_indices, output)

    def online_out(self, logits, token_ids, output):
        return self.out(logits, token_ids, output)

    def online_fp32(self, logits, token_ids):
        return self.apply_fp32(logits, token_ids)

    def online_indexed_out(self, logits, token_ids, row_indices, output):
        return self.indexed_out(logits, token_ids, row_indices, output)

    def online_indexed_fp32(self, logits, token_ids, row_indices):
        return self.indexed_fp32(logits, token_ids, row_indices)


class _LogpFromLogitsFunction(torch.autograd.Function):
    """Differentiable fp32 selected log-prob of logits (used by the logits-fed ratio/KL op)."""

    @staticmethod
    def forward(ctx, logits, ids):
        shape = logits.shape[:-1]
        logits_2d = logits.reshape(-1, logits.size(-1)).contiguous()
        ids_1d = ids.reshape(-1).to(device=logits.device, dtype=torch.long).contiguous()
        n = logits_2d.size(0)
        out = torch.empty(n, device=logits.device, dtype=torch.float32)
        lse = torch.empty(n, device=logits.device, dtype=torch.float32)
        logp_from_logits(logits_2d, ids_1d, out, lse_out=lse)
        ctx.save_for_backward(logits_2d, ids_1d, lse)
        ctx.logits_shape = logits.shape
        return out.view(shape)

    @staticmethod
    def backward(ctx, grad_out):
        logits_2d, ids_1d, lse = ctx.saved_tensors
        lib = _native.load()
        coeff = grad_out.reshape(-1).to(torch.float32).contiguous()
        grad = torch.empty_like(logits_2d)
        n, v = logits_2d.shape
        with torch.cuda.device(logits_2d.device):
            rc = lib.rlk_logp_from_logits_bwd(logits_2d.data_ptr(), _IN[logits_2d.dtype],
                                              ids_1d.data_ptr(), lse.data_ptr(), coeff.data_ptr(),
                                              grad.data_ptr(), n, v, _stream(logits_2d.device))
        _native.check(rc, "rlk_logp_from_logits_bwd")
        return grad.view(ctx.logits_shape), None


class _LogpPairFromLogitsFunction(torch.autograd.Function):
    """fp32 selected log-probs of a policy and a reference logits tensor from ONE scan launch;
    differentiable w.r.t. the policy logits only."""

    @staticmethod
    def forward(ctx, logits, ref_logits, ids):
        shape = logits.shape[:-1]
        logits_2d = logits.reshape(-1, logits.size(-1)).contiguous()
        ref_2d = ref_logits.reshape(-1, ref_logits.size(-1)).contiguous()
        ids_1d = ids.reshape(-1).to(device=logits.device, dtype=torch.long).contiguous()
        n, v = logits_2d.shape
        out = torch.empty(n, device=logits.device, dtype=torch.float32)
        ref_out = torch.empty(n, device=logits.device, dtype=torch.float32)
        lse = torch.empty(n, device=logits.device, dtype=torch.float32)
        if n > 0:
            with torch.cuda.device(logits_2d.device):
                rc = _native.load().rlk_logp_from_logits_pair(
                    logits_2d.data_ptr(), ref_2d.data_ptr(), _IN[logits_2d.dtype], ids_1d.data_ptr(),
                    out.data_ptr(), ref_out.data_ptr(), _OUT[torch.float32], lse.data_ptr(), None, None,
                    n, n, v, _stream(logits_2d.device))
            _native.check(rc, "rlk_logp_from_logits_pair")
        ctx.save_for_backward(logits_2d, ids_1d, lse)
        ctx.logits_shape = logits.shape
        ref_view = ref_out.view(shape)
        ctx.mark_non_differentiable(ref_view)
        return out.view(shape), ref_view

    @staticmethod
    def backward(ctx, grad_out, _grad_ref):
        grad, _ = _LogpFromLogitsFunction.backward(ctx, grad_out)
        return grad, None, None


def differentiable_logp_pair_fp32(logits: torch.Tensor, ref_logits: torch.Tensor,
                                  ids: torch.Tensor):
    """``(logp_policy, logp_ref)``; one launch when both tensors share shape, dtype and device,
    two scans otherwise."""
    if logits.dtype not in _IN or ref_logits.dtype not in _IN:
        raise RuntimeError("logits dtype must be float32, float16 or bfloat16")
    if (logits.shape == ref_logits.shape and logits.dtype == ref_logits.dtype
            and logits.device == ref_logits.device):
        return _LogpPairFromLogitsFunction.apply(logits, ref_logits.detach(), ids)
    with torch.no_grad():
        ref = _LogpFromLogitsFunction.apply(ref_logits.detach(), ids)
    return _LogpFromLogitsFunction.apply(logits, ids), ref


def differentiable_logp_fp32(logits: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    if logits.dtype not in _IN:
        raise RuntimeError("logits dtype must be float32, float16 or bfloat16")
    return _LogpFromLogitsFunction.apply(logits, ids)
