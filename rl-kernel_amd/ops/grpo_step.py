"""The GRPO step from hidden states in as few launches as the math allows.

``RocmFusedGRPOStepOp`` chains what the reference's trainer runs as separate steps
(rl_engine/executors/deepspeed_trainer.py:146-167: ``_extract_logps`` -> ``compute_policy_ratio`` /
``compute_reference_kl`` -> ``masked_mean``): the fused linear log-prob forward whose last launch
(the merge of the vocab splits) already emits the per-token ratio / clip / KL terms, their
fixed-order partial sums and ``d loss / d logp``; the backward feeds that gradient straight into
the recompute-based dH / dW kernels.  Values equal ``RocmFusedLinearLogpOp`` followed by
``RocmGRPOFromLogpOp`` bit for bit.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import _native
from ..platform import logger
from . import linear_logp as LL

IGNORE_INDEX = -100


@_native.on_tensor_device
def fused_linear_logp_grpo_forward(hidden_2d, weight, target_1d, bias, old, ref, adv, mask, *,
                                   seq_len: int, clip_eps: float, beta: float,
                                   temperature: float = 1.0, ignore_index: Optional[int] = None,
                                   want_grad: bool = True, want_terms: bool = False):
    """Raw launch set of ``rlk_linear_logp_fwd_grpo``; all per-token tensors are flat ``[N]``
    fp32 (``mask`` bool / uint8, ``adv`` per token ``[N]`` or per sequence ``[N / seq_len]``).
    Returns ``(logp, lse, err, out3, ratio, kl_terms, d_cur, d_kl)``."""
    lib = _native.load()
    n, h = hidden_2d.shape
    v = weight.size(0)
    dev = hidden_2d.device
    dt = LL._DTYPES[hidden_2d.dtype]
    f32 = lambda t: None if t is None else t.detach().to(device=dev, dtype=torch.float32).contiguous().reshape(-1)
    old_f, ref_f, adv_f = f32(old), f32(ref), f32(adv)
    if old_f.numel() != n or (ref_f is not None and ref_f.numel() != n):
        raise ValueError("old_logps / ref_logps must hold one value per token")
    if adv_f.numel() == n:
        per_token = 1
    elif adv_f.numel() * seq_len == n:
        per_token = 0
    else:
        raise ValueError(f"advantages with {adv_f.numel()} values match neither {n} tokens nor "
                         f"{n // max(seq_len, 1)} sequences")
    mask_u8 = None
    if mask is not None:
        if mask.numel() != n:
            raise ValueError("mask must hold one value per token")
        mask_u8 = mask.to(device=dev, dtype=torch.bool).contiguous().view(torch.uint8).reshape(-1)
    logp = torch.empty(n, device=dev, dtype=torch.float32)
    lse = torch.empty(n, device=dev, dtype=torch.float32)
    err = torch.zeros(1, device=dev, dtype=torch.int32)
    out3 = torch.empty(3, device=dev, dtype=torch.float32)
    new = lambda want: torch.empty(n, device=dev, dtype=torch.float32) if want else None
    ratio, klt, dcur, dkl = new(want_terms), new(want_terms), new(want_grad), new(want_grad)
    need = _native.ctypes.c_size_t(0)
    _native.check(lib.rlk_linear_logp_fwd_grpo_workspace_bytes(n, h, v, dt, _native.ctypes.byref(need)),
                  "fused forward + GRPO workspace query")
    ws = torch.empty(need.value, device=dev, dtype=torch.uint8)
    bias_f = None if bias is None else bias.detach().to(torch.float32).contiguous()
    p = LL._ptr
    rc = lib.rlk_linear_logp_fwd_grpo(
        p(hidden_2d), p(weight), p(bias_f), p(target_1d), p(logp), p(lse), p(ws), ws.numel(), n, h, v,
        0, dt, float(temperature), 0 if ignore_index is None else int(ignore_index),
        int(ignore_index is not None), 1, p(err), p(old_f), p(ref_f), p(adv_f), per_token,
        p(mask_u8), max(int(seq_len), 1), float(clip_eps), float(beta), p(out3), p(ratio), p(klt),
        p(dcur), p(dkl), LL._stream(dev))
    _native.check(rc, "rlk_linear_logp_fwd_grpo")
    return logp, lse, err, out3, ratio, klt, dcur, dkl


class _FusedGRPOStepFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, bias, marked_ids, old, ref, adv, mask, clip_eps, beta,
                temperature, check_targets):
        hidden_2d = LL._aligned_contiguous(hidden.reshape(-1, hidden.size(-1)))
        w = LL._aligned_contiguous(weight)
        target_1d = marked_ids.reshape(-1).to(device=hidden_2d.device, dtype=torch.long).contiguous()
        seq_len = hidden.shape[-2] if hidden.dim() >= 2 else 1
        logp, lse, err, out3, _, _, dcur, dkl = fused_linear_logp_grpo_forward(
            hidden_2d, w, target_1d, bias, old, ref, adv, mask, seq_len=seq_len, clip_eps=clip_eps,
            beta=beta, temperature=temperature, ignore_index=IGNORE_INDEX)
        if check_targets and bool(err.item()):
            raise LL._out_of_range_error(target_1d, w.size(0), IGNORE_INDEX)
        ctx.save_for_backward(hidden_2d, w, bias if bias is not None else hidden_2d, target_1d, lse,
                              dcur, dkl)
        ctx.has_bias = bias is not None
        ctx.lead_shape = hidden.shape[:-1]
        ctx.temperature = temperature
        ctx.beta = beta
        ctx.weight_dtype = weight.dtype
        ctx.bias_dtype = bias.dtype if bias is not None else None
        cur = logp.reshape(hidden.shape[:-1])
        ctx.mark_non_differentiable(cur)
        return out3[0], out3[1], out3[2], cur

    @staticmethod
    def backward(ctx, g_loss, g_pol, g_kl, _g_cur):
        hidden_2d, w, bias_t, target_1d, lse, dcur, dkl = ctx.saved_tensors
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_b = ctx.has_bias and ctx.needs_input_grad[2]
        # d loss / d logp and d kl / d logp were left by the forward; policy = loss - beta * kl
        upstream = dcur * (g_loss + g_pol) + dkl * (g_kl - ctx.beta * g_pol)
        d_h, d_w, d_b = LL.fused_linear_logp_backward(
            upstream, hidden_2d, w, target_1d, lse, bias_t if ctx.has_bias else None,
            temperature=ctx.temperature, ignore_index=IGNORE_INDEX, need_hidden=need_h,
            need_weight=need_w, need_bias=need_b)
        grad_hidden = d_h.reshape(tuple(ctx.lead_shape) + (hidden_2d.size(1),)) if need_h else None
        grad_weight = d_w.to(ctx.weight_dtype) if need_w else None
        grad_bias = d_b.to(ctx.bias_dtype) if need_b else None
        return (grad_hidden, grad_weight, grad_bias) + (None,) * 9


class RocmFusedGRPOStepOp:
    """``(loss, policy_loss, kl, current_logps)`` from hidden states ``[B, T, H]``, the lm_head
    weight, token ids / completion mask ``[B, T]``, old / reference log-probs ``[B, T]`` and
    advantages (``[B]`` per sequence or ``[B, T]`` per token).  The three scalars are
    differentiable w.r.t. hidden, weight and bias; masked positions have log-prob exactly 0 and
    no gradient."""

    def __init__(self) -> None:
        if not torch.cuda.is_available() or getattr(torch.version, "hip", None) is None:
            raise RuntimeError("RocmFusedGRPOStepOp needs a ROCm GPU")
        _native.load()
        logger.info("Linked to librlk_hip.so fused linear_logp + GRPO epilogue kernels.")

    def __call__(self, hidden, lm_head_weight, token_ids, completion_mask, old_logps, ref_logps,
                 advantages, bias=None, *, clip_eps: float = 0.2, beta: float = 0.0,
                 temperature: float = 1.0, check_targets: bool = True):
        return self.apply(hidden, lm_head_weight, token_ids, completion_mask, old_logps, ref_logps,
                          advantages, bias, clip_eps=clip_eps, beta=beta, temperature=temperature,
                          check_targets=check_targets)

    def apply(self, hidden, lm_head_weight, token_ids, completion_mask, old_logps, ref_logps,
              advantages, bias=None, *, clip_eps: float = 0.2, beta: float = 0.0,
              temperature: float = 1.0, check_targets: bool = True):
        if temperature <= 0.0:
            raise ValueError("temperature must be greater than zero")
        if hidden.dim() < 2 or hidden.shape[:-1] != token_ids.shape:
            raise ValueError(f"hidden leading shape {tuple(hidden.shape[:-1])} must match "
                             f"token_ids shape {tuple(token_ids.shape)}")
        if lm_head_weight.size(-1) != hidden.size(-1):
            raise ValueError(f"hidden dim {hidden.size(-1)} must match lm_head_weight dim "
                             f"{lm_head_weight.size(-1)}")
        if not LL.hip_path_supported(hidden, lm_head_weight):
            raise NotImplementedError("RocmFusedGRPOStepOp needs hidden and weight of one dtype "
                                      "(bf16, f16 or f32) on one GPU")
        ids = token_ids.to(device=hidden.device).long()
        mask = None
        if completion_mask is not None:
            if completion_mask.shape != token_ids.shape:
                raise ValueError(f"mask shape {tuple(completion_mask.shape)} must match token_ids "
                                 f"shape {tuple(token_ids.shape)}")
            mask = completion_mask.to(device=hidden.device, dtype=torch.bool)
            ids = ids.masked_fill(~mask, IGNORE_INDEX)
        return _FusedGRPOStepFunction.apply(hidden, lm_head_weight, bias, ids, old_logps, ref_logps,
                                            advantages, mask, float(clip_eps), float(beta),
                                            float(temperature), check_targets)
