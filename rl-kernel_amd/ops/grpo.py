"""GRPO / PPO loss on MI355X: the log-prob-fed fused epilogue and the logits-fed op classes.

* ``RocmGRPOFromLogpOp`` -- the epilogue fed by ``linear_logp``: ratio, clipped surrogate, k3 KL,
  masked token-mean and dloss/dlogp in three tiny launches
  (composition of rl_engine/testing/reference_ops.py:50-106 as chained by
  rl_engine/executors/deepspeed_trainer.py:160-167 in the reference).
* ``RocmRatioKLOp`` / ``RocmGRPOLossOp`` -- the logits-fed signatures of
  rl_engine/kernels/ops/pytorch/loss/ratio_kl.py:13-58 and
  rl_engine/kernels/ops/pytorch/loss/grpo_loss.py:13-206, built on the HIP logits scan.
"""

from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch

from .. import _native
from ..platform import logger
from .logp import differentiable_logp_pair_fp32


def _stream(device):
    return torch.cuda.current_stream(device).cuda_stream


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.detach().to(torch.float32).contiguous()


def _require_gpu(name: str) -> None:
    if not torch.cuda.is_available() or getattr(torch.version, "hip", None) is None:
        raise RuntimeError(f"{name} needs a ROCm GPU")
    _native.load()


@_native.on_tensor_device
def grpo_from_logp_raw(cur, old, ref, adv, mask, *, clip_eps, beta, want_grad, want_terms=False,
                       upstream=None):
    """One launch set of the epilogue; returns ``(out3, ratio, kl_terms, d_cur, d_kl)``."""
    lib = _native.load()
    dev = cur.device
    cur_f = _f32(cur).reshape(-1)
    n = cur_f.numel()
    seq_len = cur.shape[-1] if cur.dim() >= 1 and cur.numel() else 1
    old_f = _f32(old).reshape(-1)
    ref_f = None if ref is None else _f32(ref).reshape(-1)
    adv_f = _f32(adv)
    if adv_f.numel() == n and adv.shape == cur.shape:
        per_token = 1
    elif adv_f.numel() * seq_len == n:
        per_token = 0
    else:
        raise ValueError(f"advantages shape {tuple(adv.shape)} matches neither the token shape "
                         f"{tuple(cur.shape)} nor its leading (per-sequence) shape")
    adv_f = adv_f.reshape(-1)
    mask_u8 = None
    if mask is not None:
        if mask.shape != cur.shape:
            raise ValueError(f"mask shape {tuple(mask.shape)} must match logp shape")
        mask_u8 = mask.to(device=dev, dtype=torch.bool).contiguous().view(torch.uint8).reshape(-1)
    if old_f.numel() != n or (ref_f is not None and ref_f.numel() != n):
        raise ValueError("old_logps / ref_logps must have the shape of the current logps")
    out3 = torch.empty(3, device=dev, dtype=torch.float32)
    ratio = torch.empty(n, device=dev, dtype=torch.float32) if want_terms else None
    klt = torch.empty(n, device=dev, dtype=torch.float32) if want_terms else None
    dcur = torch.empty(n, device=dev, dtype=torch.float32) if want_grad else None
    dkl = torch.empty(n, device=dev, dtype=torch.float32) if want_grad else None
    need = _native.ctypes.c_size_t(0)
    _native.check(lib.rlk_grpo_loss_workspace_bytes(n, _native.ctypes.byref(need)), "grpo workspace")
    ws = torch.empty(need.value, device=dev, dtype=torch.uint8)
    p = lambda t: None if t is None else t.data_ptr()
    rc = lib.rlk_grpo_loss_from_logp(
        p(cur_f), p(old_f), p(ref_f), p(adv_f), per_token, p(mask_u8), n, max(int(seq_len), 1),
        float(clip_eps), float(beta), p(out3), p(ratio), p(klt), p(dcur), p(dkl), p(upstream),
        p(ws), ws.numel(), _stream(dev))
    _native.check(rc, "rlk_grpo_loss_from_logp")
    shape = cur.shape
    return (out3, None if ratio is None else ratio.view(shape),
            None if klt is None else klt.view(shape), None if dcur is None else dcur.view(shape),
            None if dkl is None else dkl.view(shape))


class _GRPOFromLogpFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, cur, old, ref, adv, mask, clip_eps, beta):
        out3, _, _, dcur, dkl = grpo_from_logp_raw(cur, old, ref, adv, mask, clip_eps=clip_eps,
                                                   beta=beta, want_grad=True)
        ctx.save_for_backward(dcur, dkl)
        ctx.cur_dtype = cur.dtype
        ctx.beta = beta
        return out3[0], out3[1], out3[2]

    @staticmethod
    def backward(ctx, g_loss, g_pol, g_kl):
        dcur, dkl = ctx.saved_tensors  # d loss / d cur and d kl / d cur
        grad = dcur * (g_loss + g_pol) + dkl * (g_kl - ctx.beta * g_pol)
        return grad.to(ctx.cur_dtype), None, None, None, None, None, None


@_native.on_tensor_device
def group_advantages(rewards: torch.Tensor, *, samples_per_prompt: Optional[int] = None,
                     group_boundaries=None, eps: float = 1e-6) -> torch.Tensor:
    """Group-normalised advantages on the GPU; argument policy of
    rl_engine/kernels/ops/pytorch/loss/grpo_loss.py:170-206 (reference)."""
    lib = _native.load()
    flat = _f32(rewards).reshape(-1)
    b = flat.numel()
    if (samples_per_prompt is None) == (group_boundaries is None):
        raise ValueError("Provide exactly one of samples_per_prompt or group_boundaries.")
    if samples_per_prompt is not None:
        if samples_per_prompt < 2:
            raise ValueError("samples_per_prompt must be at least 2 for group normalization.")
        if b % samples_per_prompt != 0:
            raise ValueError(f"num_sequences ({b}) must be divisible by "
                             f"samples_per_prompt ({samples_per_prompt}).")
        bounds = torch.arange(0, b + 1, samples_per_prompt, device=flat.device, dtype=torch.long)
    else:
        bounds_host = torch.as_tensor(group_boundaries, dtype=torch.long).cpu()
        if bounds_host.ndim != 1 or bounds_host.numel() < 2:
            raise ValueError("group_boundaries must be a 1D tensor of length num_groups + 1.")
        sizes = bounds_host[1:] - bounds_host[:-1]
        if int(bounds_host[0]) != 0 or int(sizes.sum()) != b:
            raise ValueError(f"group sizes sum to {int(sizes.sum())} but there are {b} sequences.")
        if bool((sizes < 1).any()):
            raise ValueError("each group must contain at least one sequence.")
        bounds = bounds_host.to(flat.device)
    adv = torch.empty_like(flat)
    rc = lib.rlk_group_advantages(flat.data_ptr(), bounds.data_ptr(), bounds.numel() - 1, float(eps),
                                  adv.data_ptr(), _stream(flat.device))
    _native.check(rc, "rlk_group_advantages")
    return adv


class RocmGRPOFromLogpOp:
    """Fused log-prob-fed GRPO loss: ``(loss, policy_loss, kl)``; ``loss`` is differentiable
    w.r.t. ``current_logps``.  ``advantages`` is per token ``[B, T]`` or per sequence ``[B]``."""

    def __init__(self) -> None:
        _require_gpu("RocmGRPOFromLogpOp")
        logger.info("Linked to librlk_hip.so GRPO epilogue kernels.")

    def __call__(self, current_logps, old_logps, ref_logps, advantages, completion_mask=None, *,
                 clip_eps: float = 0.2, beta: float = 0.0):
        return self.apply(current_logps, old_logps, ref_logps, advantages, completion_mask,
                          clip_eps=clip_eps, beta=beta)

    def apply(self, current_logps, old_logps, ref_logps, advantages, completion_mask=None, *,
              clip_eps: float = 0.2, beta: float = 0.0):
        return _GRPOFromLogpFunction.apply(current_logps, old_logps, ref_logps, advantages,
                                           completion_mask, float(clip_eps), float(beta))

    def ratio_and_kl(self, current_logps, old_logps, ref_logps, completion_mask=None):
        """Per-token ``(ratio, kl)`` with masked entries 0 (reference_ops.py:82-106)."""
        zeros = torch.zeros(current_logps.shape, device=current_logps.device)
        _, ratio, kl, _, _ = grpo_from_logp_raw(current_logps, old_logps, ref_logps, zeros,
                                             completion_mask, clip_eps=0.2, beta=0.0,
                                             want_grad=False, want_terms=True)
        return ratio, kl

    group_advantages = staticmethod(group_advantages)


class _RatioKLFromLogpFunction(torch.autograd.Function):
    """``(ratio, kl)`` per token from current / reference / old log-probs, one launch each way;
    differentiable w.r.t. the current log-probs only."""

    @staticmethod
    def forward(ctx, cur, ref, old, mask):
        shape = cur.shape
        dev = cur.device
        cur_f, ref_f, old_f = (_f32(t).reshape(-1) for t in (cur, ref, old))
        mask_u8 = mask.to(device=dev, dtype=torch.bool).contiguous().view(torch.uint8).reshape(-1)
        n = cur_f.numel()
        ratio = torch.empty(n, device=dev, dtype=torch.float32)
        kl = torch.empty(n, device=dev, dtype=torch.float32)
        with torch.cuda.device(dev):
            rc = _native.load().rlk_ratio_kl_from_logp(
                cur_f.data_ptr(), ref_f.data_ptr(), old_f.data_ptr(), mask_u8.data_ptr(), n,
                ratio.data_ptr(), kl.data_ptr(), _stream(dev))
        _native.check(rc, "rlk_ratio_kl_from_logp")
        ctx.save_for_backward(cur_f, ref_f, old_f, mask_u8)
        ctx.shape = shape
        return ratio.view(shape), kl.view(shape)

    @staticmethod
    def backward(ctx, g_ratio, g_kl):
        cur_f, ref_f, old_f, mask_u8 = ctx.saved_tensors
        n = cur_f.numel()
        gr = None if g_ratio is None else _f32(g_ratio).reshape(-1)
        gk = None if g_kl is None else _f32(g_kl).reshape(-1)
        d_cur = torch.empty(n, device=cur_f.device, dtype=torch.float32)
        p = lambda t: None if t is None else t.data_ptr()
        with torch.cuda.device(cur_f.device):
            rc = _native.load().rlk_ratio_kl_from_logp_bwd(
                cur_f.data_ptr(), ref_f.data_ptr(), old_f.data_ptr(), mask_u8.data_ptr(), p(gr), p(gk),
                n, d_cur.data_ptr(), _stream(cur_f.device))
        _native.check(rc, "rlk_ratio_kl_from_logp_bwd")
        return d_cur.view(ctx.shape), None, None, None


class RocmRatioKLOp:
    """Logits-fed ratio + k3 KL: mask-before-exp, so inactive positions give ratio 1 and kl 0
    (rl_engine/kernels/ops/pytorch/loss/ratio_kl.py:32-58 of the reference)."""

    def __init__(self) -> None:
        _require_gpu("RocmRatioKLOp")

    def __call__(self, policy_logits, ref_logits, action_ids, attention_mask, old_logps):
        return self.forward(policy_logits, ref_logits, action_ids, attention_mask, old_logps)

    def forward(self, policy_logits, ref_logits, action_ids, attention_mask, old_logps
                ) -> Tuple[torch.Tensor, torch.Tensor]:
        mask = attention_mask.to(torch.bool)
        vocab = policy_logits.size(-1)
        invalid = mask & ((action_ids < 0) | (action_ids >= vocab))
        if bool(invalid.any()):
            raise ValueError(f"action_ids at active (unmasked) positions must be in "
                             f"[0, {vocab}); found out-of-range ids.")
        safe_ids = action_ids.masked_fill(~mask, 0)
        # both logit tensors in one scan launch (the reference's program reads both rows too:
        # rl_engine/kernels/ops/triton/loss/ratio_kl.py:46-60)
        logp_policy, logp_ref = differentiable_logp_pair_fp32(policy_logits, ref_logits, safe_ids)
        return _RatioKLFromLogpFunction.apply(logp_policy, logp_ref, old_logps, mask)


class RocmGRPOLossOp:
    """Logits-fed GRPO loss with the reference op's signature
    (rl_engine/kernels/ops/pytorch/loss/grpo_loss.py:24-157): the selected log-probs come from
    the HIP logits scan, the loss and its gradient from the fused log-prob-fed epilogue."""

    def __init__(self) -> None:
        _require_gpu("RocmGRPOLossOp")
        self._from_logp = RocmGRPOFromLogpOp()

    def __call__(self, policy_logits, ref_logits, action_ids, old_logps, rewards, completion_mask, *,
                 clip_eps: float = 0.2, beta: float = 0.0, samples_per_prompt: Optional[int] = None,
                 group_boundaries: Optional[Sequence[int] | torch.Tensor] = None, eps: float = 1e-6):
        return self.forward(policy_logits, ref_logits, action_ids, old_logps, rewards,
                            completion_mask, clip_eps=clip_eps, beta=beta,
                            samples_per_prompt=samples_per_prompt,
                            group_boundaries=group_boundaries, eps=eps)

    def group_advantages(self, rewards, *, samples_per_prompt=None, group_boundaries=None,
                         eps: float = 1e-6):
        return group_advantages(rewards, samples_per_prompt=samples_per_prompt,
                                group_boundaries=group_boundaries, eps=eps)

    @staticmethod
    def expand_advantages(sample_advantages, completion_mask):
        bool_mask = completion_mask.bool()
        expanded = sample_advantages.reshape(-1, 1).expand_as(bool_mask).clone()
        return expanded.masked_fill(~bool_mask, 0.0)

    def apply(self, policy_logits, ref_logits, action_ids, old_logps, sample_advantages,
              completion_mask, *, clip_eps: float = 0.2, beta: float = 0.0):
        mask = completion_mask.to(torch.bool)
        vocab = policy_logits.size(-1)
        if bool((mask & ((action_ids < 0) | (action_ids >= vocab))).any()):
            raise ValueError(f"action_ids at active (unmasked) positions must be in "
                             f"[0, {vocab}); found out-of-range ids.")
        safe_ids = action_ids.masked_fill(~mask, 0)
        cur, ref = differentiable_logp_pair_fp32(policy_logits, ref_logits, safe_ids)
        return self._from_logp(cur, old_logps, ref, sample_advantages.reshape(-1), mask,
                               clip_eps=clip_eps, beta=beta)

    def forward(self, policy_logits, ref_logits, action_ids, old_logps, rewards, completion_mask, *,
                clip_eps: float = 0.2, beta: float = 0.0, samples_per_prompt=None,
                group_boundaries=None, eps: float = 1e-6):
        adv = self.group_advantages(rewards, samples_per_prompt=samples_per_prompt,
                                    group_boundaries=group_boundaries, eps=eps)
        return self.apply(policy_logits, ref_logits, action_ids, old_logps, adv, completion_mask,
                          clip_eps=clip_eps, beta=beta)
