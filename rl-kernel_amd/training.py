"""Caller-side glue of the fused path: what a training step does around the two fused ops.

Mirrors, for the one-GPU case, the part of ``DeepSpeedTrainingWorker.train`` that chains
``linear_logp`` -> ratio / clip / KL -> masked mean (rl_engine/executors/deepspeed_trainer.py:
146-169 of the reference) and its helpers: hidden-state discovery in a model output
(``_extract_hidden_states``, :424-434 with :461-556), ``_safe_token_ids`` (:559-569), the
model-input id check (:572-581), the ZeRO-3 gather of the head's parameters around the op
(``_linear_logp_parameter_context``, :584-615) and ``_extract_logps`` (:618-641).  With the HIP
backend the masking passes collapse into kernel arguments (``ignore_index``) and the epilogue into
one fused op.
"""

from __future__ import annotations

from collections.abc import Mapping
from contextlib import nullcontext
from dataclasses import dataclass
from typing import Any, Optional

import torch

IGNORE_INDEX = -100

_DIRECT_NAMES = ("last_hidden_state", "hidden")
_STACK_NAME = "hidden_states"


class ParameterGatherUnavailableError(RuntimeError):
    """ZeRO-3 partitions the head's parameters and the runtime offers no way to gather them."""


def _field(container: Any, name: str):
    """``(present, value)`` of a mapping key or an object attribute."""
    if isinstance(container, Mapping):
        return (name in container), container.get(name)
    return hasattr(container, name), getattr(container, name, None)


def _is_hidden(t: Any, dim: Optional[int]) -> bool:
    return (isinstance(t, torch.Tensor) and t.ndim >= 2
            and (dim is None or int(t.size(-1)) == int(dim)))


def _names_hidden_state(item: Any) -> bool:
    return not isinstance(item, torch.Tensor) and any(
        _field(item, n)[0] for n in _DIRECT_NAMES + (_STACK_NAME,))


def _from_stack(stack: Any, dim: Optional[int]) -> Optional[torch.Tensor]:
    """Per-layer hidden states: the last entry that holds a hidden tensor (a bare tensor counts as
    a stack of one)."""
    if isinstance(stack, torch.Tensor):
        return stack if _is_hidden(stack, dim) else None
    if isinstance(stack, (tuple, list)):
        for entry in reversed(stack):
            found = _find_hidden(entry, dim)
            if found is not None:
                return found
    return None


def _find_hidden(out: Any, dim: Optional[int]) -> Optional[torch.Tensor]:
    if isinstance(out, torch.Tensor):
        return out if _is_hidden(out, dim) else None
    if out is None:
        return None
    # named fields first: the final hidden state wins over the per-layer stack
    for name in _DIRECT_NAMES:
        present, value = _field(out, name)
        if present:
            found = _find_hidden(value, dim)
            if found is not None:
                return found
    present, value = _field(out, _STACK_NAME)
    if present:
        found = _from_stack(value, dim)
        if found is not None:
            return found
    if isinstance(out, Mapping) or not isinstance(out, (tuple, list)):
        return None
    # a plain sequence (loss, logits, hidden, ...): structured members, then an unambiguous tensor
    for item in out:
        if _names_hidden_state(item):
            found = _find_hidden(item, dim)
            if found is not None:
                return found
    tensors = [t for t in out if _is_hidden(t, dim)]
    if len(tensors) == 1:
        return tensors[0]
    if tensors:
        top = max(t.ndim for t in tensors)
        deepest = [t for t in tensors if t.ndim == top]
        if len(deepest) == 1:
            return deepest[0]
    for item in out:
        if not isinstance(item, torch.Tensor):
            found = _find_hidden(item, dim)
            if found is not None:
                return found
    return None


def extract_hidden_states(model_output: Any, *, expected_hidden_dim: Optional[int] = None
                          ) -> torch.Tensor:
    """The final hidden-state tensor of a model output, with the reference's acceptance rules
    (rl_engine/executors/deepspeed_trainer.py:424-434, 461-556): a tensor of rank >= 2 (whose last
    dimension is ``expected_hidden_dim`` when given); ``last_hidden_state`` / ``hidden`` keys or
    attributes; the last entry of ``hidden_states``; in a plain tuple a structured member, else the
    single tensor that fits (the one of highest rank when several fit).  ``TypeError`` otherwise."""
    found = _find_hidden(model_output, expected_hidden_dim)
    if found is None:
        raise TypeError("model output does not expose a hidden-state tensor: "
                        f"{type(model_output)!r}")
    return found


def validate_model_input_token_ids(token_ids: torch.Tensor, *, vocab_size: int) -> None:
    """Ids fed to the model must be real vocabulary entries; sentinels such as -100 belong to the
    log-prob / loss stage only (rl_engine/executors/deepspeed_trainer.py:572-581)."""
    bad = (token_ids < 0) | (token_ids >= int(vocab_size))
    if bool(bad.any().item()):
        raise ValueError(
            f"model input token_ids must be in [0, {int(vocab_size) - 1}], got "
            f"[{int(token_ids.min().item())}, {int(token_ids.max().item())}]. Keep ignore-index / "
            "padding sentinels out of the model input path and apply masking only at the "
            "logprob/loss stage.")


def linear_logp_parameter_context(deepspeed_runtime: Any, model: torch.nn.Module, *,
                                  zero_stage: int, world_size: int):
    """Context in which ``model.lm_head``'s weight and bias are whole tensors, which the fused op
    needs: nothing to do below ZeRO stage 3 or on one rank, otherwise the runtime's
    ``zero.GatheredParameters`` over exactly those parameters, read-only
    (rl_engine/executors/deepspeed_trainer.py:584-615)."""
    if int(zero_stage) < 3 or int(world_size) <= 1:
        return nullcontext()
    lm_head = getattr(model, "lm_head", None)
    if not isinstance(lm_head, torch.nn.Linear):
        raise TypeError("model must expose an lm_head torch.nn.Linear for ZeRO-3 linear_logp "
                        "gathering")
    gather = getattr(getattr(deepspeed_runtime, "zero", None), "GatheredParameters", None)
    if not callable(gather):
        raise ParameterGatherUnavailableError(
            "ZeRO-3 linear_logp training requires deepspeed.zero.GatheredParameters or an "
            "equivalent full-parameter gather API.")
    params = [lm_head.weight] + ([lm_head.bias] if lm_head.bias is not None else [])
    return gather(params, modifier_rank=None)


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


def extract_logps(hidden: Any, lm_head: torch.nn.Module, token_ids: torch.Tensor,
                  completion_mask: Optional[torch.Tensor], linear_logp_op: Any, *,
                  temperature: float = 1.0, output_dtype: torch.dtype = torch.float32,
                  skip_masked: bool = True) -> torch.Tensor:
    """Selected-token log-probs of ``lm_head(hidden)`` with masked positions exactly 0.

    ``hidden`` is the hidden-state tensor or any model output ``extract_hidden_states`` accepts;
    ``lm_head`` is the head (``torch.nn.Linear``) or, as in the reference's ``_extract_logps``, the
    model that exposes it as ``.lm_head``.  With an op that understands ``ignore_index`` (the HIP
    backend) masked positions are marked ``-100``; with ``skip_masked`` the op then runs its
    kernels on the unmasked rows only (``compact_ignored``: the same values to fp32 rounding,
    the masked share of the work saved), without it they pass through the kernels as rows that
    produce 0 and no gradient.  With any other ``linear_logp`` backend the reference's two-pass
    convention is used (safe ids, then ``masked_fill``)."""
    if not isinstance(lm_head, torch.nn.Linear):
        lm_head = getattr(lm_head, "lm_head", None)
    if not isinstance(lm_head, torch.nn.Linear):
        raise TypeError("model must expose an lm_head torch.nn.Linear for linear_logp")
    hidden = extract_hidden_states(hidden, expected_hidden_dim=int(lm_head.in_features))
    ids = token_ids.to(device=hidden.device)
    from .ops.linear_logp import RocmFusedLinearLogpOp

    fused = isinstance(linear_logp_op, RocmFusedLinearLogpOp)
    if fused:
        marked = ids.long()
        if completion_mask is not None:
            active = completion_mask.to(device=ids.device, dtype=torch.bool)
            marked = marked.masked_fill(~active, IGNORE_INDEX)
        logps = linear_logp_op(hidden, lm_head.weight, marked, lm_head.bias,
                               temperature=temperature, ignore_index=IGNORE_INDEX,
                               compact_ignored=skip_masked and completion_mask is not None)
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
                   registry=None, fuse_epilogue: bool = True,
                   skip_masked: bool = False) -> GRPOStepResult:
    """hidden -> fused logp -> group-normalised advantages -> fused GRPO loss (call
    ``result.loss.backward()`` for dH / dW / db).  Ops come from the kernel registry.  With
    ``fuse_epilogue`` (hidden states and head of one dtype on the GPU) the loss terms leave the
    forward's last launch (``grpo_step_from_hidden``); the values are the same bits either way.
    ``skip_masked`` takes the positions outside ``completion_mask`` out of the head's kernels
    (see ``extract_logps``; the loss then comes from the stand-alone epilogue): the step gets
    cheaper by about the masked share of the batch, and the values agree to fp32 rounding."""
    if registry is None:
        from .registry import kernel_registry as registry
    linear_logp = registry.get_op("linear_logp")
    loss_op = registry.get_op("grpo_loss_from_logp")
    if not isinstance(lm_head, torch.nn.Linear):
        lm_head = getattr(lm_head, "lm_head", None)
    if not isinstance(lm_head, torch.nn.Linear):
        raise TypeError("model must expose an lm_head torch.nn.Linear for linear_logp")
    hidden = extract_hidden_states(hidden, expected_hidden_dim=int(lm_head.in_features))
    fusable = (fuse_epilogue and not (skip_masked and completion_mask is not None)
               and hidden.dim() >= 2 and lm_head.weight.dtype == hidden.dtype
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
                        temperature=temperature, skip_masked=skip_masked)
    adv = loss_op.group_advantages(rewards, samples_per_prompt=samples_per_prompt,
                                   group_boundaries=group_boundaries)
    loss, pol, kl = loss_op(cur, old_logps, ref_logps, adv, completion_mask, clip_eps=clip_eps,
                            beta=beta)
    return GRPOStepResult(loss, pol, kl, cur, adv)
