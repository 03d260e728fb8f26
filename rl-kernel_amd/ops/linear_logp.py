"""Fused linear -> selected-token log-prob on MI355X.

``RocmFusedLinearLogpOp`` has the call signature of the reference's ``linear_logp`` backends
(rl_engine/kernels/ops/pytorch/loss/linear_logp.py:455-486,
rl_engine/kernels/ops/cuda/loss/linear_logp.py:252-359) and is differentiable w.r.t. hidden,
weight and bias.  Two keyword-only extensions with neutral defaults fold the caller-side
conventions of rl_engine/testing/reference_ops.py:15-47 into the kernel: ``temperature`` and
``ignore_index``.
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from .. import _compiled, _native
from ..platform import logger

_DTYPES = {torch.bfloat16: _native.DTYPE_BF16, torch.float16: _native.DTYPE_F16,
           torch.float32: _native.DTYPE_F32}


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _aligned_contiguous(t: torch.Tensor) -> torch.Tensor:
    t = t.contiguous()
    if t.data_ptr() % 16:
        t = t.clone(memory_format=torch.contiguous_format)
    return t


def _out_of_range_error(target_1d: torch.Tensor, vocab: int, ignore_index: Optional[int]):
    live = target_1d if ignore_index is None else target_1d[target_1d != ignore_index]
    t_min, t_max = int(live.min()), int(live.max())
    return ValueError(
        f"target_ids out of range: expected [0, {vocab - 1}], got [{t_min}, {t_max}]. "
        "Mask or filter padding / ignore-index values (e.g. -100) before this op."
    )


def _check_grad_buffer(name: str, buf: torch.Tensor, shape, device) -> None:
    if buf.dtype != torch.float32 or tuple(buf.shape) != tuple(shape) or not buf.is_contiguous() \
            or buf.device != device:
        raise ValueError(f"{name} must be a contiguous float32 tensor of shape {tuple(shape)} on "
                         f"{device}, got {buf.dtype} {tuple(buf.shape)} on {buf.device}")
    if buf.requires_grad:
        raise ValueError(f"{name} must not require grad (it is a gradient buffer)")


def _compact_rows(hidden: torch.Tensor, target_ids: torch.Tensor, ignore_index: int):
    """``(rows, hidden[rows], targets[rows])`` for the rows whose target is not ``ignore_index``,
    or ``None`` when no row or every row would be kept (then there is nothing to gain, and an
    empty block would cut the result off the autograd graph).  ``rows`` (flat indices) is filled up
    to a multiple of 256 with ignored rows, which cost a fraction of a tile and keep the block on
    the kernels' full-tile routes; they come back as the zeros they are."""
    flat = target_ids.reshape(-1).to(device=hidden.device)
    keep = flat != ignore_index
    rows = torch.nonzero(keep).squeeze(1)  # synchronises: the count sizes the launches
    n_keep = rows.numel()
    if n_keep == 0 or n_keep == flat.numel():
        return None
    fill = min(-n_keep % 256, flat.numel() - n_keep)
    if fill:
        rows = torch.cat([rows, torch.nonzero(~keep).squeeze(1)[:fill]])
    hidden_2d = hidden.reshape(-1, hidden.size(-1))
    return rows, hidden_2d.index_select(0, rows), flat.index_select(0, rows)


def hip_path_supported(hidden: torch.Tensor, weight: torch.Tensor) -> bool:
    """bf16 / f16 / f32 tensors of one dtype on one GPU.  bf16/f16 with a hidden size that is a
    multiple of 8 run on the 16-bit MFMA tiles, the rest on the fp32 matrix-core kernels."""
    return (
        hidden.is_cuda
        and weight.is_cuda
        and hidden.device == weight.device
        and hidden.dtype in _DTYPES
        and weight.dtype == hidden.dtype
    )


def _common_dtype(hidden: torch.Tensor, weight: torch.Tensor):
    """Hidden states and weight of different supported dtypes (an fp32 head over bf16 activations,
    say) are both widened to fp32, which is exact, and run on the fp32 kernels; autograd casts the
    gradients back.  The reference's portable ops upcast the same way
    (rl_engine/kernels/ops/pytorch/loss/linear_logp.py:17-22)."""
    if hidden.dtype != weight.dtype and hidden.dtype in _DTYPES and weight.dtype in _DTYPES:
        return hidden.float(), weight.float()
    return hidden, weight


_wide_path_warned = False


def _warn_if_wide_path(hidden_2d: torch.Tensor, weight: torch.Tensor) -> None:
    """The 16-bit MFMA tiles take bf16/f16 with H % 8 == 0 and 16-byte aligned matrices; 16-bit
    inputs that miss that run on the fp32 matrix instruction at roughly a tenth of the rate.  Say so
    once when a large problem ends up there."""
    global _wide_path_warned
    if _wide_path_warned or hidden_2d.dtype == torch.float32:
        return
    n, h = hidden_2d.shape
    on_mfma = (h % 8 == 0 and hidden_2d.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)
    if not on_mfma and n * h * weight.size(0) > (1 << 33):
        _wide_path_warned = True
        logger.warning(
            "linear_logp: %s inputs with H=%d run on the fp32 matrix-core kernels (the 16-bit MFMA "
            "path takes H %% 8 == 0 and 16-byte aligned matrices); expect this %d x %d x %d problem "
            "to run at about a tenth of the 16-bit rate", str(hidden_2d.dtype), h, n, h,
            weight.size(0))


@_native.on_tensor_device
def fused_linear_logp_forward(
    hidden_2d: torch.Tensor,
    weight: torch.Tensor,
    target_1d: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    *,
    temperature: float = 1.0,
    ignore_index: Optional[int] = None,
    vocab_start: int = 0,
    strict_targets: bool = True,
):
    """Raw forward: returns ``(logp, lse, err_flag)`` fp32 / fp32 / int32[1] device tensors.

    Stand-in for ``_C.fused_linear_logp_sm90`` (csrc/cuda/fused_linear_logp_sm90.cu:305-381 of the
    reference) with int64 global targets.  Does not synchronise; ``err_flag`` is non-zero when
    ``strict_targets`` and some non-ignored target lies outside the weight shard.
    """
    lib = _native.load()
    n, h = hidden_2d.shape
    v = weight.size(0)
    dev = hidden_2d.device
    compiled = _compiled.module()
    if compiled is not None and n > 0 and hidden_2d.is_contiguous() and weight.is_contiguous() \
            and target_1d.dtype == torch.long and target_1d.is_contiguous():
        # same C ABI through the compiled binding: no per-argument ctypes marshalling
        _warn_if_wide_path(hidden_2d, weight)
        logp, lse, err = compiled.fused_linear_logp_forward_ex(
            hidden_2d, weight, target_1d, bias, float(temperature), ignore_index, int(vocab_start),
            bool(strict_targets))
        return logp, lse, err
    logp = torch.empty(n, device=dev, dtype=torch.float32)
    lse = torch.empty(n, device=dev, dtype=torch.float32)
    err = torch.zeros(1, device=dev, dtype=torch.int32)
    if n == 0:  # nothing to launch
        return logp, lse, err
    _warn_if_wide_path(hidden_2d, weight)
    need = _native.ctypes.c_size_t(0)
    dt = _DTYPES[hidden_2d.dtype]
    _native.check(lib.rlk_linear_logp_fwd_workspace_bytes(n, h, v, dt, _native.ctypes.byref(need)),
                  "linear_logp workspace query")
    ws = torch.empty(max(need.value, 16), device=dev, dtype=torch.uint8)
    bias_f = None if bias is None else bias.detach().to(torch.float32).contiguous()
    rc = lib.rlk_linear_logp_fwd(
        _ptr(hidden_2d), _ptr(weight), _ptr(bias_f), _ptr(target_1d), _ptr(logp), _ptr(lse),
        _ptr(ws), ws.numel(), n, h, v, int(vocab_start), dt, float(temperature),
        0 if ignore_index is None else int(ignore_index), int(ignore_index is not None),
        int(strict_targets), _ptr(err), _stream(dev))
    _native.check(rc, "rlk_linear_logp_fwd")
    return logp, lse, err


@_native.on_tensor_device
def fused_linear_logp_forward_pair(
    hidden_2d: torch.Tensor,
    weight: torch.Tensor,
    ref_weight: torch.Tensor,
    target_1d: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    ref_bias: Optional[torch.Tensor] = None,
    *,
    temperature: float = 1.0,
    ignore_index: Optional[int] = None,
    vocab_start: int = 0,
    strict_targets: bool = True,
):
    """Policy head and frozen reference head in one launch: ``(logp, lse, ref_logp, ref_lse,
    err_flag)``, each pair equal bit for bit to ``fused_linear_logp_forward`` on that head."""
    lib = _native.load()
    n, h = hidden_2d.shape
    v = weight.size(0)
    if ref_weight.shape != weight.shape or ref_weight.dtype != weight.dtype:
        raise ValueError(f"reference weight {tuple(ref_weight.shape)} {ref_weight.dtype} must match "
                         f"the policy weight {tuple(weight.shape)} {weight.dtype}")
    dev = hidden_2d.device
    outs = [torch.empty(n, device=dev, dtype=torch.float32) for _ in range(4)]
    err = torch.zeros(1, device=dev, dtype=torch.int32)
    if n == 0:
        return (*outs, err)
    _warn_if_wide_path(hidden_2d, weight)
    need = _native.ctypes.c_size_t(0)
    dt = _DTYPES[hidden_2d.dtype]
    _native.check(lib.rlk_linear_logp_fwd_pair_workspace_bytes(n, h, v, dt, _native.ctypes.byref(need)),
                  "linear_logp pair workspace query")
    ws = torch.empty(max(need.value, 16), device=dev, dtype=torch.uint8)
    f32 = lambda b: None if b is None else b.detach().to(torch.float32).contiguous()
    bias_f, ref_bias_f = f32(bias), f32(ref_bias)
    rc = lib.rlk_linear_logp_fwd_pair(
        _ptr(hidden_2d), _ptr(weight), _ptr(ref_weight), _ptr(bias_f), _ptr(ref_bias_f),
        _ptr(target_1d), _ptr(outs[0]), _ptr(outs[1]), _ptr(outs[2]), _ptr(outs[3]), _ptr(ws),
        ws.numel(), n, h, v, int(vocab_start), dt, float(temperature),
        0 if ignore_index is None else int(ignore_index), int(ignore_index is not None),
        int(strict_targets), _ptr(err), _stream(dev))
    _native.check(rc, "rlk_linear_logp_fwd_pair")
    return (*outs, err)


@_native.on_tensor_device
def fused_norm_linear_logp_forward(
    x_2d: torch.Tensor,
    gain: torch.Tensor,
    weight: torch.Tensor,
    target_1d: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    *,
    eps: float = 1e-6,
    temperature: float = 1.0,
    ignore_index: Optional[int] = None,
):
    """Raw forward from UN-normalised hidden states: ``(logp, lse, err_flag)`` of
    ``linear_logp(rmsnorm(x, gain, eps), weight, bias)``; the normalised rows live only in the
    call's workspace."""
    lib = _native.load()
    n, h = x_2d.shape
    v = weight.size(0)
    dev = x_2d.device
    logp = torch.empty(n, device=dev, dtype=torch.float32)
    lse = torch.empty(n, device=dev, dtype=torch.float32)
    err = torch.zeros(1, device=dev, dtype=torch.int32)
    if n == 0:
        return logp, lse, err
    _warn_if_wide_path(x_2d, weight)
    gain = _aligned_contiguous(gain.detach().to(torch.float32))  # the library takes an fp32 gain
    need = _native.ctypes.c_size_t(0)
    dt = _DTYPES[x_2d.dtype]
    _native.check(lib.rlk_linear_logp_rmsnorm_fwd_workspace_bytes(n, h, v, dt, _native.ctypes.byref(need)),
                  "norm + linear_logp workspace query")
    ws = torch.empty(max(need.value, 256), device=dev, dtype=torch.uint8)
    bias_f = None if bias is None else bias.detach().to(torch.float32).contiguous()
    rc = lib.rlk_linear_logp_rmsnorm_fwd(
        _ptr(x_2d), _ptr(gain), float(eps), _ptr(weight), _ptr(bias_f), _ptr(target_1d), _ptr(logp),
        _ptr(lse), _ptr(ws), ws.numel(), n, h, v, 0, dt, float(temperature),
        0 if ignore_index is None else int(ignore_index), int(ignore_index is not None), 1,
        _ptr(err), _stream(dev))
    _native.check(rc, "rlk_linear_logp_rmsnorm_fwd")
    return logp, lse, err


@_native.on_tensor_device
def fused_norm_linear_logp_backward(
    grad_logp: torch.Tensor,
    x_2d: torch.Tensor,
    gain: torch.Tensor,
    weight: torch.Tensor,
    target_1d: torch.Tensor,
    lse: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    *,
    eps: float = 1e-6,
    temperature: float = 1.0,
    ignore_index: Optional[int] = None,
    need_x: bool = True,
    need_gain: bool = True,
    need_weight: bool = True,
    need_bias: bool = True,
    dz_budget_bytes: int = 0,
):
    """Raw backward: ``(d_x [N,H] input dtype, d_gain [H] fp32, d_weight [V,H] fp32, d_bias [V]
    fp32)``; ``d_x`` is the gradient w.r.t. the UN-normalised hidden states."""
    lib = _native.load()
    n, h = x_2d.shape
    v = weight.size(0)
    dev = x_2d.device
    dt = _DTYPES[x_2d.dtype]
    gain = _aligned_contiguous(gain.detach().to(torch.float32))  # the library takes an fp32 gain
    g = grad_logp.reshape(-1).to(torch.float32).contiguous()
    d_x = torch.empty_like(x_2d) if need_x else None
    d_gain = torch.empty(h, device=dev, dtype=torch.float32) if need_gain else None
    d_weight = torch.empty(v, h, device=dev, dtype=torch.float32) if need_weight else None
    want_bias = bias is not None and need_bias
    d_bias = torch.empty(v, device=dev, dtype=torch.float32) if want_bias else None
    bias_f = None if bias is None else bias.detach().to(torch.float32).contiguous()
    need = _native.ctypes.c_size_t(0)
    _native.check(lib.rlk_linear_logp_rmsnorm_bwd_workspace_bytes(n, h, v, dt, int(dz_budget_bytes),
                                                                  _native.ctypes.byref(need)),
                  "norm + linear_logp backward workspace query")
    ws = torch.empty(max(need.value, 256), device=dev, dtype=torch.uint8)
    rc = lib.rlk_linear_logp_rmsnorm_bwd(
        _ptr(g), _ptr(x_2d), _ptr(gain), float(eps), _ptr(weight), _ptr(bias_f), _ptr(target_1d),
        _ptr(lse), _ptr(d_x), _ptr(d_gain), _ptr(d_weight), _ptr(d_bias), _ptr(ws), ws.numel(),
        int(dz_budget_bytes), n, h, v, 0, dt, float(temperature),
        0 if ignore_index is None else int(ignore_index), int(ignore_index is not None), _stream(dev))
    _native.check(rc, "rlk_linear_logp_rmsnorm_bwd")
    return d_x, d_gain, d_weight, d_bias


@_native.on_tensor_device
def fused_linear_logp_backward(
    grad_logp: torch.Tensor,
    hidden_2d: torch.Tensor,
    weight: torch.Tensor,
    target_1d: torch.Tensor,
    lse: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    *,
    temperature: float = 1.0,
    ignore_index: Optional[int] = None,
    vocab_start: int = 0,
    need_hidden: bool = True,
    need_weight: bool = True,
    need_bias: bool = True,
    dz_budget_bytes: int = 0,
    weight_grad_out: Optional[torch.Tensor] = None,
    bias_grad_out: Optional[torch.Tensor] = None,
    accumulate: bool = False,
):
    """Raw backward: ``(d_hidden [N,H] input dtype, d_weight [V,H] fp32, d_bias [V] fp32)``.

    Stand-in for ``chunked_linear_logp_backward``
    (rl_engine/kernels/ops/pytorch/loss/linear_logp.py:383-439 of the reference); unlike it, the
    saved ``lse`` is used (as the vocab-parallel backward does, :313).

    ``weight_grad_out`` / ``bias_grad_out``: caller-owned fp32 ``[V,H]`` / ``[V]`` buffers that
    receive the gradients instead of fresh tensors (they are what the call returns);
    ``accumulate`` adds to what they hold instead of overwriting it, as the reference keeps one
    fp32 ``grad_w`` over its token chunks (same file :404,423-437).
    """
    lib = _native.load()
    n, h = hidden_2d.shape
    v = weight.size(0)
    dev = hidden_2d.device
    dt = _DTYPES[hidden_2d.dtype]
    want_bias = bias is not None and need_bias
    if weight_grad_out is not None:
        _check_grad_buffer("weight_grad_out", weight_grad_out, (v, h), dev)
    if bias_grad_out is not None:
        _check_grad_buffer("bias_grad_out", bias_grad_out, (v,), dev)
    if accumulate and ((need_weight and weight_grad_out is None) or (want_bias and bias_grad_out is None)):
        raise ValueError("accumulate=True needs the buffers to add to (weight_grad_out / bias_grad_out)")
    compiled = _compiled.module()
    if compiled is not None and hidden_2d.is_contiguous() and weight.is_contiguous() \
            and target_1d.dtype == torch.long and target_1d.is_contiguous() \
            and lse.dtype == torch.float32 and lse.is_contiguous():
        d_hidden, d_weight, d_bias = compiled.fused_linear_logp_backward(
            grad_logp, hidden_2d, weight, target_1d, lse, bias, float(temperature), ignore_index,
            int(vocab_start), bool(need_hidden), bool(need_weight), bool(want_bias),
            int(dz_budget_bytes), weight_grad_out, bias_grad_out, bool(accumulate))
        return d_hidden, d_weight, d_bias
    g = grad_logp.reshape(-1).to(torch.float32).contiguous()
    d_hidden = torch.empty_like(hidden_2d) if need_hidden else None
    d_weight = None
    if need_weight:
        d_weight = weight_grad_out if weight_grad_out is not None else \
            torch.empty(v, h, device=dev, dtype=torch.float32)
    d_bias = None
    if want_bias:
        d_bias = bias_grad_out if bias_grad_out is not None else \
            torch.empty(v, device=dev, dtype=torch.float32)
    bias_f = None if bias is None else bias.detach().to(torch.float32).contiguous()
    need = _native.ctypes.c_size_t(0)
    _native.check(lib.rlk_linear_logp_bwd_workspace_bytes(n, h, v, dt, int(dz_budget_bytes),
                                                          _native.ctypes.byref(need)),
                  "linear_logp backward workspace query")
    ws = torch.empty(need.value, device=dev, dtype=torch.uint8)
    rc = lib.rlk_linear_logp_bwd_accum(
        _ptr(g), _ptr(hidden_2d), _ptr(weight), _ptr(bias_f), _ptr(target_1d), _ptr(lse),
        _ptr(d_hidden), _ptr(d_weight), _ptr(d_bias), _ptr(ws), ws.numel(), int(dz_budget_bytes),
        n, h, v, int(vocab_start), dt, float(temperature),
        0 if ignore_index is None else int(ignore_index), int(ignore_index is not None),
        int(bool(accumulate)), _stream(dev))
    _native.check(rc, "rlk_linear_logp_bwd_accum")
    return d_hidden, d_weight, d_bias


class _FusedLinearLogpFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, bias, target_ids, temperature, ignore_index, check_targets,
                weight_grad_out=None, bias_grad_out=None, accumulate=True):
        hidden_2d = _aligned_contiguous(hidden.reshape(-1, hidden.size(-1)))
        w = _aligned_contiguous(weight)
        target_1d = target_ids.reshape(-1).to(device=hidden_2d.device, dtype=torch.long).contiguous()
        ctx.empty = hidden_2d.size(0) == 0
        ctx.weight_grad_out, ctx.bias_grad_out, ctx.accumulate = weight_grad_out, bias_grad_out, accumulate
        if ctx.empty:  # no tokens: nothing to launch, gradients are zeros
            ctx.save_for_backward(hidden_2d, w, bias if bias is not None else hidden_2d, target_1d,
                                  hidden_2d.new_zeros(0, dtype=torch.float32))
            ctx.has_bias = bias is not None
            ctx.lead_shape = hidden.shape[:-1]
            ctx.weight_dtype = weight.dtype
            ctx.bias_dtype = bias.dtype if bias is not None else None
            return hidden_2d.new_zeros(hidden.shape[:-1], dtype=torch.float32)
        logp, lse, err = fused_linear_logp_forward(
            hidden_2d, w, target_1d, bias, temperature=temperature, ignore_index=ignore_index)
        if check_targets and bool(err.item()):
            raise _out_of_range_error(target_1d, w.size(0), ignore_index)
        ctx.save_for_backward(hidden_2d, w, bias if bias is not None else hidden_2d, target_1d, lse)
        ctx.has_bias = bias is not None
        ctx.lead_shape = hidden.shape[:-1]
        ctx.temperature = temperature
        ctx.ignore_index = ignore_index
        ctx.weight_dtype = weight.dtype
        ctx.bias_dtype = bias.dtype if bias is not None else None
        return logp.reshape(hidden.shape[:-1])

    @staticmethod
    def backward(ctx, grad_logp):
        hidden_2d, w, bias_t, target_1d, lse = ctx.saved_tensors
        need_h, need_w, need_b = ctx.needs_input_grad[0], ctx.needs_input_grad[1], \
            ctx.has_bias and ctx.needs_input_grad[2]
        w_out = getattr(ctx, "weight_grad_out", None)
        b_out = getattr(ctx, "bias_grad_out", None)
        accumulate = getattr(ctx, "accumulate", True)
        nones = (None,) * 7
        if ctx.empty:
            # no tokens: the gradients are zeros; buffers that accumulate stay as they are
            if w_out is not None and not accumulate:
                w_out.zero_()
            if b_out is not None and not accumulate:
                b_out.zero_()
            return (hidden_2d.new_zeros(tuple(ctx.lead_shape) + (hidden_2d.size(1),)) if need_h else None,
                    torch.zeros_like(w, dtype=ctx.weight_dtype) if need_w and w_out is None else None,
                    torch.zeros_like(bias_t, dtype=ctx.bias_dtype) if need_b and b_out is None else None,
                    *nones)
        # a caller-owned buffer receives its gradient even when the parameter itself is frozen for
        # autograd (main-grad trainers detach their parameters' .grad handling)
        want_w = need_w or w_out is not None
        want_b = ctx.has_bias and (need_b or b_out is not None)
        adding = accumulate and (w_out is not None or b_out is not None)
        w_buf, b_buf = w_out, b_out
        if adding:
            # one switch covers both buffers in the library: a gradient without a caller buffer
            # gets a zeroed one here, so that adding to it is the same as writing it
            if want_w and w_buf is None:
                w_buf = torch.zeros(w.shape, device=w.device, dtype=torch.float32)
            if want_b and b_buf is None:
                b_buf = torch.zeros(w.size(0), device=w.device, dtype=torch.float32)
        d_h, d_w, d_b = fused_linear_logp_backward(
            grad_logp, hidden_2d, w, target_1d, lse, bias_t if ctx.has_bias else None,
            temperature=ctx.temperature, ignore_index=ctx.ignore_index,
            need_hidden=need_h, need_weight=want_w, need_bias=want_b,
            weight_grad_out=w_buf, bias_grad_out=b_buf, accumulate=adding)
        grad_hidden = d_h.reshape(tuple(ctx.lead_shape) + (hidden_2d.size(1),)) if need_h else None
        grad_weight = d_w.to(ctx.weight_dtype) if need_w and w_out is None else None
        grad_bias = d_b.to(ctx.bias_dtype) if need_b and b_out is None else None
        return (grad_hidden, grad_weight, grad_bias, *nones)


class _FusedNormLinearLogpFunction(torch.autograd.Function):
    """linear_logp(rmsnorm(x, gain)) from the un-normalised hidden states; saves x, not the
    normalised rows."""

    @staticmethod
    def forward(ctx, x, gain, weight, bias, target_ids, eps, temperature, ignore_index, check_targets):
        x_2d = _aligned_contiguous(x.reshape(-1, x.size(-1)))
        g = _aligned_contiguous(gain.detach().to(torch.float32))  # the reference multiplies by weight.float()
        w = _aligned_contiguous(weight)
        target_1d = target_ids.reshape(-1).to(device=x_2d.device, dtype=torch.long).contiguous()
        logp, lse, err = fused_norm_linear_logp_forward(
            x_2d, g, w, target_1d, bias, eps=eps, temperature=temperature, ignore_index=ignore_index)
        ctx.empty = x_2d.size(0) == 0
        if check_targets and not ctx.empty and bool(err.item()):
            raise _out_of_range_error(target_1d, w.size(0), ignore_index)
        ctx.save_for_backward(x_2d, g, w, bias if bias is not None else x_2d, target_1d, lse)
        ctx.has_bias = bias is not None
        ctx.lead_shape = x.shape[:-1]
        ctx.eps, ctx.temperature, ctx.ignore_index = eps, temperature, ignore_index
        ctx.gain_dtype, ctx.weight_dtype = gain.dtype, weight.dtype
        ctx.bias_dtype = bias.dtype if bias is not None else None
        return logp.reshape(x.shape[:-1])

    @staticmethod
    def backward(ctx, grad_logp):
        x_2d, g, w, bias_t, target_1d, lse = ctx.saved_tensors
        need_x, need_g, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.needs_input_grad[2]
        need_b = ctx.has_bias and ctx.needs_input_grad[3]
        if ctx.empty:
            return (torch.zeros(tuple(ctx.lead_shape) + (x_2d.size(1),), device=x_2d.device,
                                dtype=x_2d.dtype) if need_x else None,
                    torch.zeros_like(g, dtype=ctx.gain_dtype) if need_g else None,
                    torch.zeros_like(w, dtype=ctx.weight_dtype) if need_w else None,
                    torch.zeros_like(bias_t, dtype=ctx.bias_dtype) if need_b else None,
                    None, None, None, None, None)
        d_x, d_g, d_w, d_b = fused_norm_linear_logp_backward(
            grad_logp, x_2d, g, w, target_1d, lse, bias_t if ctx.has_bias else None, eps=ctx.eps,
            temperature=ctx.temperature, ignore_index=ctx.ignore_index, need_x=need_x,
            need_gain=need_g, need_weight=need_w, need_bias=need_b)
        return (d_x.reshape(tuple(ctx.lead_shape) + (x_2d.size(1),)) if need_x else None,
                d_g.to(ctx.gain_dtype) if need_g else None,
                d_w.to(ctx.weight_dtype) if need_w else None,
                d_b.to(ctx.bias_dtype) if need_b else None, None, None, None, None, None)


class _FusedLinearLogpPairFunction(torch.autograd.Function):
    """Policy log-probs (differentiable) and reference log-probs (no gradient) from one launch."""

    @staticmethod
    def forward(ctx, hidden, weight, bias, ref_weight, ref_bias, target_ids, temperature,
                ignore_index, check_targets):
        hidden_2d = _aligned_contiguous(hidden.reshape(-1, hidden.size(-1)))
        w = _aligned_contiguous(weight)
        w_ref = _aligned_contiguous(ref_weight.detach())
        target_1d = target_ids.reshape(-1).to(device=hidden_2d.device, dtype=torch.long).contiguous()
        logp, lse, ref_logp, _, err = fused_linear_logp_forward_pair(
            hidden_2d, w, w_ref, target_1d, bias, ref_bias, temperature=temperature,
            ignore_index=ignore_index)
        if check_targets and hidden_2d.size(0) > 0 and bool(err.item()):
            raise _out_of_range_error(target_1d, w.size(0), ignore_index)
        ctx.empty = hidden_2d.size(0) == 0
        ctx.save_for_backward(hidden_2d, w, bias if bias is not None else hidden_2d, target_1d, lse)
        ctx.has_bias = bias is not None
        ctx.lead_shape = hidden.shape[:-1]
        ctx.temperature = temperature
        ctx.ignore_index = ignore_index
        ctx.weight_dtype = weight.dtype
        ctx.bias_dtype = bias.dtype if bias is not None else None
        ref_out = ref_logp.reshape(hidden.shape[:-1])
        ctx.mark_non_differentiable(ref_out)
        return logp.reshape(hidden.shape[:-1]), ref_out

    @staticmethod
    def backward(ctx, grad_logp, _grad_ref):
        grads = _FusedLinearLogpFunction.backward(ctx, grad_logp)
        return grads[0], grads[1], grads[2], None, None, None, None, None, None


class RocmFusedLinearLogpOp:
    """gfx950 MFMA fused linear log-prob: ``log_softmax((hidden W^T + b)/T)[target]`` without the
    ``[N, V]`` logits.  Constructor raises ``RuntimeError`` when the HIP library or a ROCm GPU is
    missing so that a registry can fall through to its next backend
    (rl_engine/kernels/registry.py:219-229 of the reference)."""

    def __init__(self) -> None:
        if not torch.cuda.is_available() or getattr(torch.version, "hip", None) is None:
            raise RuntimeError("RocmFusedLinearLogpOp needs a ROCm GPU")
        _native.load()
        logger.info("Linked to librlk_hip.so fused linear_logp kernels.")

    def __call__(self, hidden, lm_head_weight, target_ids, bias=None, *, tp_group: Any = None,
                 vocab_start_index: int = 0, global_vocab_size: Optional[int] = None,
                 temperature: float = 1.0, ignore_index: Optional[int] = None,
                 check_targets: bool = True, norm_weight: Optional[torch.Tensor] = None,
                 norm_eps: float = 1e-6, weight_grad_out: Optional[torch.Tensor] = None,
                 bias_grad_out: Optional[torch.Tensor] = None,
                 accumulate: bool = True, compact_ignored: bool = False) -> torch.Tensor:
        return self.apply(hidden, lm_head_weight, target_ids, bias, tp_group=tp_group,
                          vocab_start_index=vocab_start_index, global_vocab_size=global_vocab_size,
                          temperature=temperature, ignore_index=ignore_index,
                          check_targets=check_targets, norm_weight=norm_weight, norm_eps=norm_eps,
                          weight_grad_out=weight_grad_out, bias_grad_out=bias_grad_out,
                          accumulate=accumulate, compact_ignored=compact_ignored)

    def apply(self, hidden, lm_head_weight, target_ids, bias=None, *, tp_group: Any = None,
              vocab_start_index: int = 0, global_vocab_size: Optional[int] = None,
              temperature: float = 1.0, ignore_index: Optional[int] = None,
              check_targets: bool = True, norm_weight: Optional[torch.Tensor] = None,
              norm_eps: float = 1e-6, weight_grad_out: Optional[torch.Tensor] = None,
              bias_grad_out: Optional[torch.Tensor] = None, accumulate: bool = True,
              compact_ignored: bool = False) -> torch.Tensor:
        """Selected-token log-prob in float32 with the leading shape of ``hidden``.

        ``compact_ignored`` (keyword-only, default off; needs ``ignore_index``): the rows whose
        target is ``ignore_index`` (prompt and padding positions of an RL batch) are left out of
        the kernels instead of being carried through them as rows of zeros: the other rows are
        gathered into a dense ``[n_active, H]`` block, the forward and the backward run on that
        block, and the results are put back (ignored positions: log-prob 0, zero hidden gradient,
        no contribution to the weight gradient, as without the option).  Rows do not interact, so
        the results are the same numbers; they are not always the same bits, because the number of
        vocab splits, token chunks and vocab pieces follows the row count and the fp32 sums are
        then grouped differently (log-probs agree to about 1e-6, gradients to one rounding of
        their output type).  Costs one host synchronisation (the launch sizes depend on the
        count) and the gathered block, ``n_active * H`` elements held until the backward.

        ``weight_grad_out`` / ``bias_grad_out`` (keyword-only, default off): contiguous float32
        ``[V, H]`` / ``[V]`` buffers of the caller (fp32 main gradients).  The backward then adds
        the head's weight / bias gradient to them in place (``accumulate=False``: overwrites them)
        and autograd returns ``None`` for that parameter: no ``[V, H]`` temporary and no cast per
        call, and micro-batches accumulate as the reference's backward accumulates its token
        chunks into one fp32 ``grad_w``
        (rl_engine/kernels/ops/pytorch/loss/linear_logp.py:404,423-437 of the reference).

        ``norm_weight`` (keyword-only, default off): ``hidden`` is then the UN-normalised output
        of the last layer and the model's final RMSNorm
        (rl_engine/kernels/ops/pytorch/norm/rms_norm.py:54-70 of the reference, gain
        ``norm_weight``, ``norm_eps``) runs inside the op; the gradient flows to the un-normalised
        hidden states and to the gain, and the normalised activations are never kept."""
        if temperature <= 0.0:
            raise ValueError("temperature must be greater than zero")
        if lm_head_weight.size(-1) != hidden.size(-1):
            raise ValueError(
                f"hidden dim {hidden.size(-1)} must match lm_head_weight dim "
                f"{lm_head_weight.size(-1)}")
        if lm_head_weight.device != hidden.device:
            raise ValueError(
                f"lm_head_weight device {lm_head_weight.device} must match hidden "
                f"device {hidden.device}")
        if hidden.shape[:-1] != target_ids.shape:
            raise ValueError(
                f"hidden leading shape {tuple(hidden.shape[:-1])} must match "
                f"target_ids shape {tuple(target_ids.shape)}")
        vocab = lm_head_weight.size(0)
        if bias is not None:
            if bias.ndim != 1 or bias.numel() != vocab:
                raise ValueError(f"bias must be 1-D with V={vocab} elements, got "
                                 f"shape {tuple(bias.shape)}")
            if bias.device != hidden.device:
                raise ValueError(f"bias device {bias.device} must match hidden device "
                                 f"{hidden.device}")
        # Vocab-parallel metadata follows the reference's argument policy
        # (rl_engine/kernels/ops/pytorch/loss/linear_logp.py:58-83): without a multi-rank group it
        # is an error.  This build runs on one GPU; a multi-rank group is not implemented.
        if vocab <= 0:
            raise ValueError("lm_head_weight must contain at least one vocab row.")
        if tp_group is not None:
            raise NotImplementedError(
                "vocab-parallel linear_logp over a process group is not part of the one-GPU build")
        if vocab_start_index != 0:
            raise ValueError("vocab_start_index requires a tensor-parallel group.")
        if global_vocab_size is not None and int(global_vocab_size) != vocab:
            raise ValueError("global_vocab_size differs from the local vocab size, but no "
                             "multi-rank tensor-parallel group was provided.")
        if norm_weight is None:
            hidden, lm_head_weight = _common_dtype(hidden, lm_head_weight)
        if not hip_path_supported(hidden, lm_head_weight):
            raise NotImplementedError(
                "RocmFusedLinearLogpOp needs hidden and lm_head_weight in bf16, f16 or f32 on the "
                "same GPU (and of one dtype when norm_weight is given)")
        for name, buf, shape in (("weight_grad_out", weight_grad_out, tuple(lm_head_weight.shape)),
                                 ("bias_grad_out", bias_grad_out, (vocab,))):
            if buf is not None:
                _check_grad_buffer(name, buf, shape, hidden.device)
        if bias_grad_out is not None and bias is None:
            raise ValueError("bias_grad_out given without a bias")
        if compact_ignored and ignore_index is not None:
            compact = _compact_rows(hidden, target_ids, ignore_index)
            if compact is not None:
                rows, hidden_c, target_c = compact
                logp_c = self.apply(hidden_c, lm_head_weight, target_c, bias, temperature=temperature,
                                    ignore_index=ignore_index, check_targets=check_targets,
                                    norm_weight=norm_weight, norm_eps=norm_eps,
                                    weight_grad_out=weight_grad_out, bias_grad_out=bias_grad_out,
                                    accumulate=accumulate)
                full = logp_c.new_zeros(target_ids.numel()).index_copy(0, rows, logp_c)
                return full.reshape(target_ids.shape)
        if norm_weight is not None:
            if weight_grad_out is not None or bias_grad_out is not None:
                raise NotImplementedError("weight_grad_out / bias_grad_out are not wired into the "
                                          "norm_weight form of the op")
            if norm_weight.dim() != 1 or norm_weight.shape[0] != hidden.size(-1):
                raise ValueError(f"norm_weight must be 1-D of size hidden.shape[-1]={hidden.size(-1)}, "
                                 f"got tuple(norm_weight.shape)={tuple(norm_weight.shape)}")
            if norm_weight.device != hidden.device:
                raise ValueError(f"norm_weight device {norm_weight.device} must match hidden device "
                                 f"{hidden.device}")
            return _FusedNormLinearLogpFunction.apply(hidden, norm_weight, lm_head_weight, bias,
                                                      target_ids, float(norm_eps), float(temperature),
                                                      ignore_index, check_targets)
        return _FusedLinearLogpFunction.apply(hidden, lm_head_weight, bias, target_ids,
                                              float(temperature), ignore_index, check_targets,
                                              weight_grad_out, bias_grad_out, bool(accumulate))

    def with_reference(self, hidden, lm_head_weight, ref_lm_head_weight, target_ids, bias=None,
                       ref_bias=None, *, temperature: float = 1.0,
                       ignore_index: Optional[int] = None, check_targets: bool = True):
        """``(logp, ref_logp)``: the policy head and a frozen reference head over the same hidden
        states and targets in one launch (the reference log-probs the KL term needs, which the
        trainer otherwise gets from a second lm_head pass).  ``logp`` is differentiable w.r.t.
        hidden, weight and bias; ``ref_logp`` carries no gradient.  Each equals what ``apply``
        returns for that head, bit for bit."""
        if temperature <= 0.0:
            raise ValueError("temperature must be greater than zero")
        if lm_head_weight.size(-1) != hidden.size(-1):
            raise ValueError(f"hidden dim {hidden.size(-1)} must match lm_head_weight dim "
                             f"{lm_head_weight.size(-1)}")
        if ref_lm_head_weight.shape != lm_head_weight.shape:
            raise ValueError(f"reference weight shape {tuple(ref_lm_head_weight.shape)} must match "
                             f"lm_head_weight shape {tuple(lm_head_weight.shape)}")
        if hidden.shape[:-1] != target_ids.shape:
            raise ValueError(f"hidden leading shape {tuple(hidden.shape[:-1])} must match "
                             f"target_ids shape {tuple(target_ids.shape)}")
        if (bias is None) != (ref_bias is None):
            raise ValueError("both heads must have a bias or neither")
        if not hip_path_supported(hidden, lm_head_weight) or \
                ref_lm_head_weight.dtype != lm_head_weight.dtype or \
                ref_lm_head_weight.device != lm_head_weight.device:
            raise NotImplementedError(
                "with_reference needs hidden and both weights of one dtype (bf16, f16 or f32) on "
                "the same GPU")
        return _FusedLinearLogpPairFunction.apply(hidden, lm_head_weight, bias, ref_lm_head_weight,
                                                  ref_bias, target_ids, float(temperature),
                                                  ignore_index, check_targets)
