"""CPU oracle for the fused linear-logprob path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package may import this module; it is the checker used by
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py``.  Every function restates, with torch CPU library routines, the
algorithm of one reference function (cited as ``file:line`` relative to the
reference tree).  The library routines themselves (``F.linear``, ``log_softmax``,
``gather``, ``exp``, ``clamp``) are torch, not the reference.

How each function is pinned (see tests/test_oracle_*.py):

* ``linear_logp``              known answers of tests/test_reference_ops.py:18-28,60-71;
                               independent double-precision C restatement (rlk_oracle.c);
                               one-shot vs online (``linear_logp_online_stats``) agreement.
* ``linear_logp_online_stats`` associativity: any vocab chunking gives the same lse; 4-shard
                               partition [0,3,7,12,16] of tests/test_linear_logp.py:64-127.
* ``linear_logp_backward``     equals torch autograd of ``linear_logp`` on the tiny shapes of
                               tests/test_linear_logp.py:255-312; C restatement; chunk-size
                               independence; layout permutation invariance.
* ``logp_from_logits``         known answers above; out-of-range -> 0 rule of
                               csrc/fused_logp_kernel.cu:147-155.
* ``policy_ratio``/``reference_kl``/``masked_mean``
                               known answers tests/test_reference_ops.py:79-105.
* ``group_advantages``         rewards [1,3,10,20,30], bounds [0,2,5] ->
                               [-1,1,(x-20)/sqrt(200/3)] (tests/test_grpo_loss.py:110-117).
* ``grpo_loss_from_logp``      closed-form gradient vs torch autograd of the composition;
                               invariants of tests/test_ratio_kl.py:82-97,163-176.
* ``rms_norm``                 torch's own ``F.rms_norm`` (independent implementation, 1e-6) and the
                               hand-written fp32 formula bit for bit, batch-slice invariance
                               (tests/test_rms_norm.py:22-64 of the reference); unit-gain rows have
                               mean square 1; scaling x by a power of two leaves the output unchanged
                               up to eps.
* ``rms_norm_backward``        torch autograd of ``rms_norm`` in float64; d_x is orthogonal to x
                               when the gain is 1 and eps is 0 (the norm is scale-invariant).
"""

from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch

LOW_PRECISION = (torch.float16, torch.bfloat16)


# --------------------------------------------------------------------------- #
# linear -> logp forward
# --------------------------------------------------------------------------- #
def linear_logits(hidden_2d: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]):
    """fp32 logits on fp32-upcast operands.

    Follows rl_engine/kernels/ops/pytorch/loss/linear_logp.py:17-38 with the
    low-precision policy the reference's own tests apply to fused backends
    (tests/test_linear_logp.py:162-170: upcast everything to fp32 first).
    """
    b = None if bias is None else bias.float()
    return torch.nn.functional.linear(hidden_2d.float(), weight.float(), b)


def linear_logp(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    target_ids: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    *,
    temperature: float = 1.0,
    ignore_index: Optional[int] = None,
    return_lse: bool = False,
):
    """Selected-token log-prob ``z_t - logsumexp(z)`` with ``z = (h W^T + b) / T``.

    One-shot form of rl_engine/kernels/ops/pytorch/loss/linear_logp.py:514-520.
    Temperature and ignore-index semantics are those of
    rl_engine/testing/reference_ops.py:15-47: logits are divided by T before the
    log-softmax, ``T <= 0`` is an error, ignored positions gather id 0 and are
    forced to exactly 0.0.
    """
    if temperature <= 0.0:
        raise ValueError("temperature must be greater than zero")
    if hidden.shape[:-1] != target_ids.shape:
        raise ValueError("hidden leading shape must match target_ids shape")
    lead = hidden.shape[:-1]
    h2 = hidden.reshape(-1, hidden.size(-1))
    t1 = target_ids.reshape(-1).long()
    active = torch.ones_like(t1, dtype=torch.bool) if ignore_index is None else t1 != ignore_index
    safe = torch.where(active, t1, torch.zeros_like(t1))
    vocab = weight.size(0)
    if bool(((safe < 0) | (safe >= vocab)).any()):
        raise ValueError("target_ids out of range")
    z = linear_logits(h2, weight, bias) / float(temperature)
    lse = torch.logsumexp(z, dim=-1)
    zt = z.gather(-1, safe.unsqueeze(1)).squeeze(1)
    logp = torch.where(active, zt - lse, torch.zeros_like(lse))
    if return_lse:
        return logp.reshape(lead), lse.reshape(lead)
    return logp.reshape(lead)


def linear_logp_online_stats(
    hidden_2d: torch.Tensor,
    weight_local: torch.Tensor,
    target_1d: torch.Tensor,
    bias_local: Optional[torch.Tensor] = None,
    *,
    vocab_start: int = 0,
    vocab_chunk: int = 4096,
    temperature: float = 1.0,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Running (max, sum, target-logit, owner-count) over vocab chunks of a shard.

    Follows rl_engine/kernels/ops/pytorch/loss/linear_logp.py:167-214: per vocab
    chunk ``sum <- sum*exp(m - m') + sum_v exp(z_v - m')``; the target logit is
    captured by the chunk whose global column range holds it; targets outside the
    shard leave ``z_t = 0`` and ``owner = 0``.
    """
    n = hidden_2d.size(0)
    vl = weight_local.size(0)
    run_max = torch.full((n,), -math.inf)
    run_sum = torch.zeros(n)
    zt = torch.zeros(n)
    owner = torch.zeros(n, dtype=torch.int32)
    t = target_1d.long()
    for v0 in range(0, vl, vocab_chunk):
        v1 = min(vl, v0 + vocab_chunk)
        z = linear_logits(
            hidden_2d, weight_local[v0:v1], None if bias_local is None else bias_local[v0:v1]
        ) / float(temperature)
        new_max = torch.maximum(run_max, z.max(dim=-1).values)
        run_sum = run_sum * torch.exp(run_max - new_max) + torch.exp(z - new_max[:, None]).sum(-1)
        run_max = new_max
        g0, g1 = vocab_start + v0, vocab_start + v1
        hit = (t >= g0) & (t < g1)
        if bool(hit.any()):
            rows = torch.nonzero(hit).squeeze(1)
            zt[rows] = z[rows, t[rows] - g0]
            owner[rows] += 1
    return run_max, run_sum, zt, owner


def combine_online_stats(parts: Sequence[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]]):
    """Merge per-split ``(max, sum, z_t)`` in list order.

    Follows csrc/cuda/fused_linear_logp_sm90.cu:256-280:
    ``M = max_s m_s; S = sum_s s_s exp(m_s - M); z_t = sum_s z_t,s;
    lse = M + log S; logp = z_t - lse``.
    """
    big = torch.stack([p[0] for p in parts]).max(dim=0).values
    total = torch.zeros_like(big)
    zt = torch.zeros_like(big)
    for m, s, z in parts:
        total = total + s * torch.exp(m - big)
        zt = zt + z
    lse = big + torch.log(total)
    return zt - lse, lse


# --------------------------------------------------------------------------- #
# linear -> logp backward
# --------------------------------------------------------------------------- #
def linear_logp_backward(
    grad_logp: torch.Tensor,
    hidden: torch.Tensor,
    weight: torch.Tensor,
    target_ids: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    *,
    temperature: float = 1.0,
    ignore_index: Optional[int] = None,
    token_chunk: int = 1024,
):
    """fp32 ``(dH, dW, db)`` of ``sum(grad_logp * logp)``.

    Follows rl_engine/kernels/ops/pytorch/loss/linear_logp.py:383-439: per token
    chunk recompute logits, ``dz = g * (onehot - softmax(z)) / T``,
    ``dH = dz W``, ``dW += dz^T x``, ``db += sum_rows dz``; all matmuls in fp32 on
    upcast operands (:406,426-428).  Ignored rows carry ``g = 0``
    (rl_engine/executors/deepspeed_trainer.py:639-641 masks logp after the op, so
    no gradient reaches those rows).  Results are returned in fp32; casting to the
    input dtypes is the caller's choice.
    """
    h2 = hidden.reshape(-1, hidden.size(-1)).float()
    w = weight.float()
    t1 = target_ids.reshape(-1).long()
    g = grad_logp.reshape(-1).float()
    if ignore_index is not None:
        active = t1 != ignore_index
        g = torch.where(active, g, torch.zeros_like(g))
        t1 = torch.where(active, t1, torch.zeros_like(t1))
    n, d = h2.shape
    v = w.size(0)
    inv_t = 1.0 / float(temperature)
    d_h = torch.empty(n, d)
    d_w = torch.zeros(v, d)
    d_b = torch.zeros(v) if bias is not None else None
    for i0 in range(0, n, token_chunk):
        i1 = min(n, i0 + token_chunk)
        x = h2[i0:i1]
        z = linear_logits(x, w, bias) * inv_t
        dz = -torch.softmax(z, dim=-1)
        dz[torch.arange(i1 - i0), t1[i0:i1]] += 1.0
        dz *= (g[i0:i1] * inv_t)[:, None]
        d_h[i0:i1] = dz @ w
        d_w += dz.t() @ x
        if d_b is not None:
            d_b += dz.sum(0)
    return d_h.reshape(tuple(hidden.shape[:-1]) + (d,)), d_w, d_b


# --------------------------------------------------------------------------- #
# logits -> logp (fused_logp family)
# --------------------------------------------------------------------------- #
def logp_from_logits(
    logits: torch.Tensor,
    token_ids: torch.Tensor,
    *,
    out_of_range_is_zero: bool = True,
) -> torch.Tensor:
    """fp32 selected log-prob of materialised logits.

    Follows rl_engine/kernels/ops/pytorch/loss/logp.py:16-32 (log_softmax of the
    fp32 upcast + gather).  With ``out_of_range_is_zero`` the native rule of
    csrc/fused_logp_kernel.cu:147-155,197-205 applies: a target outside
    ``[0, V)`` yields 0 instead of an error.
    """
    v = logits.size(-1)
    l2 = logits.reshape(-1, v).float()
    t = token_ids.reshape(-1).long()
    ok = (t >= 0) & (t < v)
    if not out_of_range_is_zero and not bool(ok.all()):
        raise ValueError("token id out of range")
    lp = torch.log_softmax(l2, dim=-1).gather(-1, torch.where(ok, t, 0).unsqueeze(1)).squeeze(1)
    return torch.where(ok, lp, torch.zeros_like(lp)).reshape(logits.shape[:-1])


def logp_from_logits_indexed(logits, token_ids, row_indices, output):
    """Write only the listed rows of ``output`` (others untouched).

    Follows rl_engine/kernels/ops/pytorch/loss/logp.py:55-66 for valid rows and
    csrc/fused_logp_kernel.cu:120-123 (rows outside ``[0, N)`` are skipped).
    """
    n = logits.numel() // logits.size(-1)
    idx = row_indices.reshape(-1).long()
    idx = idx[(idx >= 0) & (idx < n)]
    vals = logp_from_logits(logits, token_ids).reshape(-1)
    flat = output.reshape(-1)
    flat[idx] = vals[idx].to(output.dtype)
    return output


# --------------------------------------------------------------------------- #
# logp-fed GRPO epilogue
# --------------------------------------------------------------------------- #
def policy_ratio(cur, old, mask=None):
    """``exp(cur - old)``, masked entries 0 (rl_engine/testing/reference_ops.py:82-92)."""
    r = torch.exp(cur.float() - old.float())
    return r if mask is None else torch.where(mask.bool(), r, torch.zeros_like(r))


def reference_kl(cur, ref, mask=None):
    """k3 estimator ``e^d - d - 1, d = ref - cur`` (reference_ops.py:95-106)."""
    d = ref.float() - cur.float()
    k = torch.exp(d) - d - 1.0
    return k if mask is None else torch.where(mask.bool(), k, torch.zeros_like(k))


def masked_mean(values, mask=None, eps: float = 1e-8):
    """``sum(values*mask) / max(count, eps)`` in fp32 (reference_ops.py:50-79)."""
    v = values.float()
    if mask is None:
        return v.sum() / max(float(v.numel()), eps)
    m = mask.bool()
    return torch.where(m, v, torch.zeros_like(v)).sum() / m.sum().float().clamp_min(eps)


def group_ids(num_sequences, samples_per_prompt=None, group_boundaries=None):
    """Sequence -> group id (rl_engine/kernels/ops/pytorch/loss/grpo_loss.py:170-206)."""
    if (samples_per_prompt is None) == (group_boundaries is None):
        raise ValueError("Provide exactly one of samples_per_prompt or group_boundaries.")
    if samples_per_prompt is not None:
        if samples_per_prompt < 2:
            raise ValueError("samples_per_prompt must be at least 2 for group normalization.")
        if num_sequences % samples_per_prompt:
            raise ValueError("num_sequences must be divisible by samples_per_prompt.")
        return torch.arange(num_sequences) // samples_per_prompt
    b = torch.as_tensor(group_boundaries, dtype=torch.long)
    if b.ndim != 1 or b.numel() < 2:
        raise ValueError("group_boundaries must be a 1D tensor of length num_groups + 1.")
    sizes = b[1:] - b[:-1]
    if int(sizes.sum()) != num_sequences:
        raise ValueError("group sizes do not sum to the number of sequences.")
    if bool((sizes < 1).any()):
        raise ValueError("each group must contain at least one sequence.")
    return torch.repeat_interleave(torch.arange(sizes.numel()), sizes)


def group_advantages(rewards, *, samples_per_prompt=None, group_boundaries=None, eps: float = 1e-6):
    """``(x - mean_g) / sqrt(max(E[x^2] - mean^2, eps^2))`` per group.

    Follows rl_engine/kernels/ops/pytorch/loss/grpo_loss.py:53-84 (population
    variance from sums of squares, floor ``eps**2`` under the square root).
    """
    x = rewards.reshape(-1).float()
    gid = group_ids(x.numel(), samples_per_prompt, group_boundaries)
    ng = int(gid.max()) + 1 if x.numel() else 0
    cnt = torch.zeros(ng).index_add_(0, gid, torch.ones_like(x))
    s1 = torch.zeros(ng).index_add_(0, gid, x)
    s2 = torch.zeros(ng).index_add_(0, gid, x * x)
    mean = s1 / cnt
    std = (s2 / cnt - mean * mean).clamp_min(eps * eps).sqrt()
    return (x - mean[gid]) / std[gid]


def grpo_loss_from_logp(
    cur_logp: torch.Tensor,
    old_logp: torch.Tensor,
    ref_logp: torch.Tensor,
    advantages: torch.Tensor,
    mask: torch.Tensor,
    *,
    clip_eps: float = 0.2,
    beta: float = 0.0,
):
    """``(loss, policy_loss, kl, dloss/dcur)`` of the logp-fed GRPO objective.

    Composition of rl_engine/testing/reference_ops.py:71-106 as chained by
    rl_engine/executors/deepspeed_trainer.py:160-167 and
    rl_engine/kernels/ops/pytorch/loss/grpo_loss.py:96-125:
    ``loss = mean_mask(-min(r A, clip(r) A)) + beta * mean_mask(k3)``.
    ``advantages`` is per token ``[B,T]`` or per sequence ``[B]``.  The gradient is
    the closed form of torch's subgradient choices: ``minimum`` sends the
    gradient to the smaller branch and splits it on ties; ``clamp`` passes it on
    the closed interval.
    """
    cur = cur_logp.float()
    m = mask.bool()
    adv = advantages.float()
    if adv.dim() == cur.dim() - 1:
        adv = adv.unsqueeze(-1).expand_as(cur)
    adv = torch.where(m, adv, torch.zeros_like(adv))
    r = policy_ratio(cur, old_logp, m)
    lo, hi = 1.0 - clip_eps, 1.0 + clip_eps
    unclipped = r * adv
    clipped = r.clamp(lo, hi) * adv
    pol_terms = -torch.minimum(unclipped, clipped)
    d = ref_logp.float() - cur
    kl_terms = torch.where(m, torch.exp(d) - d - 1.0, torch.zeros_like(d))
    denom = m.sum().float().clamp_min(1e-8)
    policy_loss = pol_terms.sum() / denom
    kl = kl_terms.sum() / denom
    loss = policy_loss + beta * kl
    inside = (r >= lo) & (r <= hi)
    w_un = torch.where(unclipped < clipped, 1.0, torch.where(unclipped == clipped, 0.5, 0.0))
    w_cl = 1.0 - w_un
    dpol = -(w_un * adv * r + w_cl * adv * r * inside.float())
    dkl = 1.0 - torch.exp(d)
    grad = torch.where(m, (dpol + beta * dkl) / denom, torch.zeros_like(cur))
    return loss, policy_loss, kl, grad


# --------------------------------------------------------------------------- #
# RMSNorm in front of the head
# --------------------------------------------------------------------------- #
def rms_norm(x: torch.Tensor, weight: torch.Tensor, *, eps: float = 1e-6,
             output_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``x * rsqrt(mean(x^2, -1) + eps) * weight`` accumulated in fp32, cast to ``x.dtype``
    (or ``output_dtype``).  Follows rl_engine/kernels/ops/pytorch/norm/rms_norm.py:54-70,
    including its ValueError for a weight that is not ``[x.shape[-1]]``."""
    if weight.dim() != 1 or weight.shape[0] != x.shape[-1]:
        raise ValueError(f"weight must be 1-D of size x.shape[-1]={x.shape[-1]}, "
                         f"got tuple(weight.shape)={tuple(weight.shape)}")
    x_f = x.float()
    var = x_f.pow(2).mean(dim=-1, keepdim=True)
    normed = x_f * torch.rsqrt(var + eps)
    out = normed * weight.float()
    return out.to(x.dtype if output_dtype is None else output_dtype)


def rms_norm_backward(grad_out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, *,
                      eps: float = 1e-6) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 ``(d_x, d_weight)`` of ``sum(grad_out * rms_norm(x, weight))``: what autograd derives
    for rl_engine/kernels/ops/pytorch/norm/rms_norm.py:66-70.  With r = rsqrt(mean(x^2) + eps)
    and g = grad_out * weight:  d_x = r g - x r^3 mean(g x),  d_weight = sum_rows grad_out x r."""
    x_f = x.float().reshape(-1, x.shape[-1])
    go = grad_out.float().reshape(-1, x.shape[-1])
    w = weight.float()
    r = torch.rsqrt(x_f.pow(2).mean(dim=-1, keepdim=True) + eps)
    g = go * w
    d_x = r * g - x_f * r.pow(3) * (g * x_f).mean(dim=-1, keepdim=True)
    d_w = (go * x_f * r).sum(dim=0)
    return d_x.reshape(x.shape), d_w
