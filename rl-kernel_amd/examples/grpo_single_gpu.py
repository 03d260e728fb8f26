#!/usr/bin/env python3
"""A whole GRPO training step on the fused ops, on one MI355X, with a toy policy.

    python rl-kernel_amd/examples/grpo_single_gpu.py --steps 4

Counterpart of the reference's examples/grpo_single_gpu.py, with one structural difference: the
policy's head is never applied as a dense layer.  The trunk's hidden states go straight into the
fused ``linear_logp`` op (no [tokens, vocab] logits in memory), masked positions are skipped inside
the kernel, and ratio / clip / KL / token-mean run as one fused op.  Every step also recomputes the
selected log-probs with plain PyTorch and prints the drift.
"""
from __future__ import annotations

import argparse
import os
import sys
from dataclasses import dataclass

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


@dataclass(frozen=True)
class StepMetrics:
    step: int
    loss: float
    policy_loss: float
    kl: float
    active_tokens: int
    max_abs_drift: float


class ToyTrunk(torch.nn.Module):
    """Embedding + one gated block + RMS normalisation; returns hidden states [B, T, H]."""

    def __init__(self, vocab: int, hidden: int):
        super().__init__()
        self.embed = torch.nn.Embedding(vocab, hidden)
        self.up = torch.nn.Linear(hidden, 2 * hidden, bias=False)
        self.down = torch.nn.Linear(hidden, hidden, bias=False)
        self.gain = torch.nn.Parameter(torch.ones(hidden))

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        x = self.embed(ids)
        a, b = self.up(x).chunk(2, dim=-1)
        x = x + self.down(torch.nn.functional.silu(a) * b)
        x = x * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6).to(x.dtype)
        return x * self.gain


def parse_args(argv=None) -> argparse.Namespace:
    p = argparse.ArgumentParser(description=__doc__)
    p.add_argument("--steps", type=int, default=4)
    p.add_argument("--num-prompts", type=int, default=2)
    p.add_argument("--samples-per-prompt", type=int, default=4)
    p.add_argument("--completion-len", type=int, default=16)
    p.add_argument("--vocab-size", type=int, default=1000)
    p.add_argument("--hidden-dim", type=int, default=64)
    p.add_argument("--dtype", choices=("bf16", "f16", "f32"), default="bf16")
    p.add_argument("--lr", type=float, default=2e-2)
    p.add_argument("--clip-eps", type=float, default=0.2)
    p.add_argument("--beta", type=float, default=0.01)
    p.add_argument("--temperature", type=float, default=1.0)
    p.add_argument("--seed", type=int, default=1234)
    return p.parse_args(argv)


def run_training(args: argparse.Namespace) -> list[StepMetrics]:
    if args.steps <= 0:
        raise ValueError("--steps must be greater than zero")
    if not torch.cuda.is_available():
        raise RuntimeError("this example runs the HIP kernels and needs a ROCm GPU")
    from rl_kernel_amd.registry import kernel_registry
    from rl_kernel_amd.training import extract_logps, grpo_loss_step

    dev = torch.device("cuda:0")
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[args.dtype]
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    torch.manual_seed(args.seed)
    b, t, v = args.num_prompts * args.samples_per_prompt, args.completion_len, args.vocab_size
    ids = torch.randint(0, v, (b, t), device=dev, generator=gen)
    lens = torch.randint(max(1, t // 2), t + 1, (b,), device=dev, generator=gen)
    mask = torch.arange(t, device=dev)[None, :] < lens[:, None]
    # reward of a sequence: mean of (token id mod 7) / 6 over its completion, as in the reference example
    rewards = ((ids.float() % 7.0) / 6.0).masked_fill(~mask, 0.0).sum(1) / lens.float()

    trunk = ToyTrunk(v, args.hidden_dim).to(dev, dtype)
    head = torch.nn.Linear(args.hidden_dim, v, bias=True).to(dev, dtype)
    params = list(trunk.parameters()) + list(head.parameters())
    opt = torch.optim.AdamW(params, lr=args.lr)
    op = kernel_registry.get_op("linear_logp")

    with torch.no_grad():
        old = extract_logps(trunk(ids), head, ids, mask, op, temperature=args.temperature)
        ref = old.clone()
    print(f"starting grpo_single_gpu backend={type(op).__name__} batch={b}x{t} "
          f"active_tokens={int(mask.sum())} dtype={args.dtype}")

    out: list[StepMetrics] = []
    for step in range(args.steps):
        opt.zero_grad(set_to_none=True)
        hidden = trunk(ids)
        res = grpo_loss_step(hidden, head, ids, mask, old, ref, rewards,
                             samples_per_prompt=args.samples_per_prompt, clip_eps=args.clip_eps,
                             beta=args.beta, temperature=args.temperature)
        if not torch.isfinite(res.loss):
            raise RuntimeError(f"non-finite loss at step {step}")
        with torch.no_grad():  # plain PyTorch recomputation of the same log-probs
            logits = torch.nn.functional.linear(hidden.float(), head.weight.float(), head.bias.float())
            plain = torch.log_softmax(logits / args.temperature, -1).gather(-1, ids[..., None])[..., 0]
            drift = (res.current_logps - plain.masked_fill(~mask, 0.0)).abs().max().item()
        res.loss.backward()
        opt.step()
        m = StepMetrics(step, res.loss.item(), res.policy_loss.item(), res.kl.item(),
                        int(mask.sum()), drift)
        out.append(m)
        print(f"step={m.step} loss={m.loss:.6f} policy_loss={m.policy_loss:.6f} kl={m.kl:.6f} "
              f"max_abs_drift={m.max_abs_drift:.3e}")
    print(f"completed grpo_single_gpu steps={args.steps}")
    return out


def main() -> None:
    run_training(parse_args())


if __name__ == "__main__":
    main()
