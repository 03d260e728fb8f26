"""Caller-side glue of the fused path: what a training step does around the two fused ops.

Mirrors, for the one-GPU case, the part of ``DeepSpeedTrainingWorker.train`` that chains
``linear_logp`` -> ratio / clip / KL -> masked mean (rl_engine/executors/deepspeed_trainer.py:
146-169 of the reference) and its helpers ``_safe_token_ids`` (:559-569) and ``_extract_logps``
(:618-641).  With the HIP backend the masking passes collapse into kernel arguments
(``ignore_index``) and the epilogue into one fused op.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

import torch

IGNORE_INDEX = -100


def safe_token_ids(token_ids: torch.Tensor, mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """int64 ids with masked positions replaced by 0 (the reference's gather-safe convention)."""
    ids = token_ids.long()
    if mask is None:
        return ids
    active = mask.to(device=ids.device, dtype=torch.bool)
    if active.shape != ids.shape:
        raise ValueError(f"mask shape {tuple(active.shape)} must match token_ids shape "
                         f"{tuple(ids.shape)}")
    return ids.masked_fill(~active, 0)


def extract_logps(hidden: torch.Tensor, lm_head: torch.nn.Linear, token_ids: torch.Tensor,
                  completion_mask: Optional[torch.Tensor], linear_logp_op: Any, *,
                  temperature: float = 1.0, output_dtype: torch.dtype = torch.float32
                  ) -> torch.Tensor:
    """Selected-token log-probs of ``lm_head(hidden)`` with masked positions exactly 0.

    With an op that understands ``ignore_index`` (the HIP backend) masked positions are marked
    ``-100`` and skipped inside the kernel; with any other ``linear_logp`` backend the
    reference's two-pass convention is used (safe ids, then ``masked_fill``)."""
    if not isinstance(lm_head, torch.nn.Linear):
        raise TypeError("model must expose an lm_head torch.nn.Linear for linear_logp")
    ids = token_ids.to(device=hidden.device)
    from .ops.linear_logp import RocmFusedLinearLogpOp

    fused = isinstance(linear_logp_op, RocmFusedLinearLogpOp)
    if fused:
        marked = ids.long()
        if completion_mask is not None:
            active = completion_mask.to(device=ids.device, dtype=torch.bool)
            marked = marked.masked_fill(~active, IGNORE_INDEX)
        logps = linear_logp_op(hidden, lm_head.weight, marked, lm_head.bias,
                               temperature=temperature, ignore_index=IGNORE_INDEX)
    else:
        if temperature != 1.0:
            raise ValueError("only the fused HIP backend takes a temperature")
        logps = linear_logp_op(hidden, lm_head.weight, safe_token_ids(ids, completion_mask),
                               lm_head.bias)
        if completion_mask is not None:
            logps = logps.masked_fill(~completion_mask.to(device=logps.device, dtype=torch.bool), 0.0)
    return logps.to(dtype=output_dtype)


@dataclass
class GRPOStepResult:
    loss: torch.Tensor
    policy_loss: torch.Tensor
    kl: torch.Tensor
    current_logps: torch.Tensor
    advantages: torch.Tensor


def grpo_loss_step(hidden: torch.Tensor, lm_head: torch.nn.Linear, token_ids: torch.Tensor,
                   completion_mask: torch.Tensor, old_logps: torch.Tensor,
                   ref_logps: Optional[torch.Tensor], rewards: torch.Tensor, *,
                   samples_per_prompt: Optional[int] = None, group_boundaries=None,
                   clip_eps: float = 0.2, beta: float = 0.0, temperature: float = 1.0,
                   registry=None, fuse_epilogue: bool = True) -> GRPOStepResult:
    """hidden -> fused logp -> group-normalised advantages -> fused GRPO loss (call
    ``result.loss.backward()`` for dH / dW / db).  Ops come from the kernel registry.  With
    ``fuse_epilogue`` (hidden states and head of one dtype on the GPU) the loss terms leave the
    forward's last launch (``grpo_step_from_hidden``); the values are the same bits either way."""
    if registry is None:
        from .registry import kernel_registry as registry
    linear_logp = registry.get_op("linear_logp")
    loss_op = registry.get_op("grpo_loss_from_logp")
    if not isinstance(lm_head, torch.nn.Linear):
        raise TypeError("model must expose an lm_head torch.nn.Linear for linear_logp")
    fusable = (fuse_epilogue and hidden.dim() >= 2 and lm_head.weight.dtype == hidden.dtype
               and hidden.dtype in (torch.bfloat16, torch.float16, torch.float32))
    if fusable:
        step_op = registry.get_op("grpo_step_from_hidden")
        adv = loss_op.group_advantages(rewards, samples_per_prompt=samples_per_prompt,
                                       group_boundaries=group_boundaries)
        loss, pol, kl, cur = step_op(hidden, lm_head.weight, token_ids, completion_mask, old_logps,
                                     ref_logps, adv, lm_head.bias, clip_eps=clip_eps, beta=beta,
                                     temperature=temperature)
        return GRPOStepResult(loss, pol, kl, cur, adv)
    cur = extract_logps(hidden, lm_head, token_ids, completion_mask, linear_logp,
                        temperature=temperature)
    adv = loss_op.group_advantages(rewards, samples_per_prompt=samples_per_prompt,
                                   group_boundaries=group_boundaries)
    loss, pol, kl = loss_op(cur, old_logps, ref_logps, adv, completion_mask, clip_eps=clip_eps,
                            beta=beta)
    return GRPOStepResult(loss, pol, kl, cur, adv)
