#!/usr/bin/env python3
"""Benchmark of the fused linear-logprob hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

One step = one forward (logp, lse) + one backward (dH in the input dtype, dW fp32) of the fused
LM-head log-prob over one synthetic batch at the Llama-3-8B head shape (32768 tokens, H=4096,
V=128256, bf16), through the C-ABI library.  Inputs are resident in HBM before the timed region.
Prints ONE JSON line (metric = tokens/s of the whole step) carrying a `roofline` object for the
dominant kernel (the forward contraction, timed with HIP events on the launch stream) and a
`cpu_baseline` object (the CPU oracle timed on a bounded token slice on the host cores).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0}  # MI355X dense MFMA, published

# HBM bytes moved by ONE forward launch of the default workload, from two `rocprofv3 --pmc` runs of
# this script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter
# reads for the 1 GiB `--calibrate-copy` kernel (factors 2.000 and 1.000):
# 2.000 * 24869400 KiB + 1.000 * 1536 KiB.  Other workloads report null.
MEASURED_FWD_TRAFFIC_BYTES = {"llama3-8b-head": (2.0 * 24869400 + 1536) * 1024}

WORKLOADS = {
    # BASELINE.json configs[1] shape; the metric is quoted on forward+backward at this shape
    "llama3-8b-head": dict(tokens=32768, hidden=4096, vocab=128256, dtype="bf16",
                           temperature=1.0, ignore_frac=0.0),
    "llama3-8b-head-64k": dict(tokens=65536, hidden=4096, vocab=128256, dtype="bf16",
                               temperature=0.7, ignore_frac=0.0),
    "qwen3-head": dict(tokens=131072, hidden=2048, vocab=151936, dtype="f16",
                       temperature=1.0, ignore_frac=0.01),
    # BASELINE.json configs[4]: the configs[1] shape with the GRPO epilogue between forward and
    # backward (one group of 64 responses x 512 positions, response lengths U{128..512})
    "llama3-8b-grpo-step": dict(tokens=32768, hidden=4096, vocab=128256, dtype="bf16",
                                temperature=1.0, ignore_frac=0.0, grpo=dict(group=64, seq=512,
                                                                            clip_eps=0.2, beta=0.04)),
    # the logits-fed `fused_logp` scan (HBM-bound): 16384 rows of Llama-3 vocabulary, bf16 logits
    "logits-scan": dict(tokens=16384, hidden=0, vocab=128256, dtype="bf16", temperature=1.0,
                        ignore_frac=0.0, scan=True),
    "small": dict(tokens=4096, hidden=1024, vocab=32768, dtype="bf16", temperature=1.0,
                  ignore_frac=0.0),
}


def make_inputs(torch, cfg, device, seed=1002):
    gen = torch.Generator(device=device).manual_seed(seed)
    dt = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float16
    n, h, v = cfg["tokens"], cfg["hidden"], cfg["vocab"]
    hidden = torch.randn(n, h, device=device, dtype=torch.float32, generator=gen).to(dt)
    weight = torch.empty(v, h, device=device, dtype=dt)
    step = 16384  # generate W in slabs to bound the fp32 temporary
    for v0 in range(0, v, step):
        v1 = min(v, v0 + step)
        weight[v0:v1] = (torch.randn(v1 - v0, h, device=device, dtype=torch.float32,
                                     generator=gen) * 0.02).to(dt)
    targets = torch.randint(0, v, (n,), device=device, generator=gen)
    if cfg["ignore_frac"] > 0:
        drop = torch.rand(n, device=device, generator=gen) < cfg["ignore_frac"]
        targets = torch.where(drop, torch.full_like(targets, -100), targets)
    grad = torch.randn(n, device=device, dtype=torch.float32, generator=gen)
    return hidden, weight, targets, grad


def cpu_baseline(torch, cfg, slice_tokens, iters=3):
    """Time the CPU oracle (fp32 linear + log_softmax + gather, closed-form backward) on a slice."""
    from oracle import oracle as O

    gen = torch.Generator().manual_seed(7)
    h, v = cfg["hidden"], cfg["vocab"]
    hidden = torch.randn(slice_tokens, h, generator=gen)
    weight = torch.randn(v, h, generator=gen) * 0.02
    targets = torch.randint(0, v, (slice_tokens,), generator=gen)
    grad = torch.randn(slice_tokens, generator=gen)

    def step():
        O.linear_logp(hidden, weight, targets, temperature=cfg["temperature"])
        O.linear_logp_backward(grad, hidden, weight, targets, temperature=cfg["temperature"],
                               token_chunk=1024)

    step()  # warm-up
    times = []
    for _ in range(iters):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": slice_tokens / med,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{slice_tokens}-token slice at the full H={h}, V={v}; fp32 torch CPU oracle "
                  f"forward+backward, 1 warm-up + {iters} timed, median; host cpu_count="
                  f"{os.cpu_count()}",
    }


def device_info(torch):
    p = torch.cuda.get_device_properties(0)
    khz = getattr(p, "clock_rate", 0)  # kHz where this torch build exposes it
    info = {"name": p.name, "compute_units": p.multi_processor_count}
    if khz:
        info["max_sclk_mhz"] = khz / 1e3
        info["peak_from_cu_clock_tflops"] = p.multi_processor_count * 4096 * khz * 1e3 / 1e12
    return info


def bench_scan(torch, args, cfg) -> int:
    """logp from materialised logits (rlk_logp_from_logits): one pass over N x V logits."""
    from rl_kernel_amd.ops.logp import logp_from_logits

    dev = torch.device("cuda:0")
    n, v = cfg["tokens"], cfg["vocab"]
    dt = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float16
    gen = torch.Generator(device=dev).manual_seed(1006)
    logits = torch.empty(n, v, device=dev, dtype=dt)
    for r0 in range(0, n, 2048):
        logits[r0:r0 + 2048] = (torch.randn(min(2048, n - r0), v, device=dev, generator=gen) * 1.3).to(dt)
    ids = torch.randint(0, v, (n,), device=dev, generator=gen)
    out = torch.empty(n, device=dev, dtype=torch.float32)
    first = logp_from_logits(logits, ids, out).clone()
    for _ in range(args.warmup):
        logp_from_logits(logits, ids, out)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        logp_from_logits(logits, ids, out)
    e1.record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    k_ms = e0.elapsed_time(e1) / args.steps
    nbytes = float(n * v * logits.element_size() + n * 8 + n * 4)
    result = {
        "metric": "logp from logits tokens/sec", "value": n / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": f"logits-scan: selected-token logp from {n} x {v} {cfg['dtype']} logits",
                   "tokens": n, "vocab": v},
        "bitwise_repeatable": bool(torch.equal(first, out)),
        "device": device_info(torch),
        "roofline": {"kernel": "logp_scan_kernel", "bound": "hbm", "achieved": nbytes / (k_ms * 1e-3) / 1e9,
                     "peak": 8000.0, "unit": "GB/s", "frac": nbytes / (k_ms * 1e-3) / 1e9 / 8000.0,
                     "traffic": None, "algorithmic_bytes": nbytes, "launch_ms": k_ms},
    }
    print(json.dumps(result))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama3-8b-head", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-slice", type=int, default=1024,
                    help="tokens of the CPU-baseline slice (0 = skip the CPU baseline)")
    ap.add_argument("--mode", default="fwd+bwd", choices=["fwd+bwd", "fwd"])
    ap.add_argument("--dtype", default=None, choices=["bf16", "f16"],
                    help="override the workload's 16-bit input type")
    ap.add_argument("--no-library-gemm", action="store_true",
                    help="skip the vendor-GEMM comparison figure")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy (known HBM traffic) so that a "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run can be scaled")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; every figure is a one-GPU figure. "
              "Run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback.", file=sys.stderr)
        return 3

    from rl_kernel_amd.ops import linear_logp as LL

    cfg = dict(WORKLOADS[args.workload])
    if args.dtype:
        cfg["dtype"] = args.dtype
    if cfg.get("scan"):
        return bench_scan(torch, args, cfg)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    hidden, weight, targets, grad = make_inputs(torch, cfg, dev)
    n, h, v = cfg["tokens"], cfg["hidden"], cfg["vocab"]
    ign = -100 if cfg["ignore_frac"] > 0 else None
    temp = cfg["temperature"]
    do_bwd = args.mode == "fwd+bwd"

    fwd_ev = []
    epi_ev = []
    grpo = cfg.get("grpo")
    if grpo:
        from rl_kernel_amd.ops import grpo as GR

        g, t = grpo["group"], grpo["seq"]
        gen = torch.Generator(device=dev).manual_seed(1005)
        lens = torch.randint(128, t + 1, (g,), device=dev, generator=gen)
        mask = torch.arange(t, device=dev)[None, :] < lens[:, None]
        targets = torch.where(mask.reshape(-1), targets, torch.full_like(targets, -100))
        ign = -100
        new_logp, _, _ = LL.fused_linear_logp_forward(hidden, weight, targets, None,
                                                      temperature=temp, ignore_index=ign)
        old = (new_logp + 0.05 * torch.randn(n, device=dev, generator=gen)).view(g, t)
        ref = (new_logp + 0.05 * torch.randn(n, device=dev, generator=gen)).view(g, t)
        rewards = torch.randn(g, device=dev, generator=gen)
        del new_logp

    def grpo_step(record):
        logp, lse, _ = LL.fused_linear_logp_forward(hidden, weight, targets, None,
                                                    temperature=temp, ignore_index=ign)
        if record:
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
        adv = GR.group_advantages(rewards, samples_per_prompt=g)
        out3, _, _, d_cur, _ = GR.grpo_from_logp_raw(logp.view(g, t), old, ref, adv, mask,
                                                     clip_eps=grpo["clip_eps"], beta=grpo["beta"],
                                                     want_grad=True)
        if record:
            e1.record()
            epi_ev.append((e0, e1))
        d_h, d_w, _ = LL.fused_linear_logp_backward(d_cur.reshape(-1), hidden, weight, targets, lse,
                                                    None, temperature=temp, ignore_index=ign)
        return (logp, lse, out3, d_h, d_w)

    def step(record=False):
        if grpo:
            return grpo_step(record)
        if record:
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
        logp, lse, err = LL.fused_linear_logp_forward(hidden, weight, targets, None,
                                                      temperature=temp, ignore_index=ign)
        if record:
            e1.record()
            fwd_ev.append((e0, e1))
        out = (logp, lse)
        if do_bwd:
            d_h, d_w, _ = LL.fused_linear_logp_backward(grad, hidden, weight, targets, lse, None,
                                                        temperature=temp, ignore_index=ign)
            out = (logp, lse, d_h, d_w)
        return out

    if args.calibrate_copy:
        src = torch.ones(1 << 28, device=dev, dtype=torch.float32)   # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        torch.neg(src, out=dst)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()
    torch.cuda.synchronize()
    base_mem = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    first = step()
    torch.cuda.synchronize()
    out_bytes = sum(t.numel() * t.element_size() for t in first)
    peak_extra = torch.cuda.max_memory_allocated() - base_mem - out_bytes
    for _ in range(max(0, args.warmup - 1)):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    last = None
    for _ in range(args.steps):
        last = step(record=True)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms = elapsed * 1e3 / args.steps

    deterministic = all(torch.equal(a, b) for a, b in zip(first, last))
    if grpo:
        # the forward launch is timed on its own after the steps (the step brackets the epilogue)
        for _ in range(3):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            LL.fused_linear_logp_forward(hidden, weight, targets, None, temperature=temp,
                                         ignore_index=ign)
            e1.record()
            fwd_ev.append((e0, e1))
        torch.cuda.synchronize()
    fwd_ms = sum(a.elapsed_time(b) for a, b in fwd_ev) / len(fwd_ev)
    fwd_flops = 2.0 * n * h * v
    achieved = fwd_flops / (fwd_ms * 1e-3) / 1e12
    peak = PEAK_TFLOPS[cfg["dtype"]]
    step_flops = (8.0 if do_bwd else 2.0) * n * h * v

    result = {
        "metric": "logp fwd+bwd tokens/sec" if do_bwd else "logp fwd tokens/sec",
        "value": n / (ms * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": cfg["dtype"],
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: fused LM-head logp {args.mode}, {n} tokens, H={h}, "
                        f"V={v}, {cfg['dtype']} in / fp32 accumulate, T={temp}",
            "tokens": n, "hidden": h, "vocab": v, "mode": args.mode,
        },
        "step_tflops": step_flops / (ms * 1e-3) / 1e12,
        "step_frac_of_mfma_peak": step_flops / (ms * 1e-3) / 1e12 / peak,
        "step_flop_accounting": "8*N*H*V (fwd 2 + logit recompute 2 + dH 2 + dW 2)" if do_bwd
                                else "2*N*H*V",
        "step_tflops_no_recompute_accounting": (6.0 if do_bwd else 2.0) * n * h * v / (ms * 1e-3) / 1e12,
        "peak_extra_hbm_bytes": int(peak_extra),
        "device": device_info(torch),
        "seed": 1002,
        "bitwise_repeatable": bool(deterministic),
        "roofline": {
            "kernel": "linear_logp_fwd_kernel",
            "bound": "mfma",
            "achieved": achieved,
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": achieved / peak,
            "traffic": MEASURED_FWD_TRAFFIC_BYTES.get(args.workload),
            "algorithmic_bytes": float((n * h + v * h) * 2 + n * 8 + n * 8),
            "launch_ms": fwd_ms,
            "flops_per_launch": fwd_flops,
        },
    }
    if not args.no_library_gemm:
        # vendor GEMM (torch.matmul -> hipBLASLt) on the same box at the same H, for scale only:
        # hidden [N, H] x W[:16384]^T -> [N, 16384] in the input dtype
        try:
            wv = weight[: min(v, 16384)]
            torch.matmul(hidden, wv.t())
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(5):
                torch.matmul(hidden, wv.t())
            e1.record()
            torch.cuda.synchronize()
            lib_ms = e0.elapsed_time(e1) / 5
            result["library_gemm"] = {
                "what": f"torch.matmul [{n},{h}] x [{h},{wv.shape[0]}] {cfg['dtype']} (writes the logits it computes)",
                "tflops": 2.0 * n * h * wv.shape[0] / (lib_ms * 1e-3) / 1e12, "ms": lib_ms}
        except Exception as exc:  # the comparison is optional
            result["library_gemm"] = {"error": str(exc)[:200]}
    if grpo:
        epi_ms = sum(a.elapsed_time(b) for a, b in epi_ev) / len(epi_ev)
        epi_bytes = n * (4 + 4 + 4 + 1 + 4 + 4)  # cur, old, ref, mask in; d_cur, d_kl out
        result["metric"] = "GRPO step (logp fwd + loss epilogue + bwd) tokens/sec"
        result["epilogue"] = {
            "bound": "hbm", "ms": epi_ms, "algorithmic_bytes": epi_bytes,
            "achieved": epi_bytes / (epi_ms * 1e-3) / 1e9, "peak": 8000.0, "unit": "GB/s",
            "frac": epi_bytes / (epi_ms * 1e-3) / 1e9 / 8000.0,
            "note": "group advantages + loss/grad launches incl. host launch gaps; 0.7 MB of "
                    "traffic, launch-latency-bound",
            "active_tokens": int(mask.sum().item()),
        }
    if args.cpu_slice > 0:
        result["cpu_baseline"] = cpu_baseline(torch, cfg, args.cpu_slice)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
