#!/usr/bin/env python3
"""Benchmark of the fused linear-logprob hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

One step = one forward (logp, lse) + one backward (dH in the input dtype, dW fp32) of the fused
LM-head log-prob over one synthetic batch at the Llama-3-8B head shape (32768 tokens, H=4096,
V=128256, bf16), through the C-ABI library.  Inputs are resident in HBM before the timed region.

Prints ONE JSON line.  Besides the headline metric (tokens/s of the whole step) it carries
  * `kernels`: the four contraction kernels of the step (forward, dZ recompute, dH, dW), each with
    its average launch time from HIP events on the launch stream, flops per launch and fraction
    of the dense bf16 MFMA peak; `roofline` is the entry of the kernel that takes the most time;
  * `through_registry_op`: the same step driven through `kernel_registry.get_op("linear_logp")`
    and autograd (adds the target-range check and the cast of dW to the weight dtype);
  * `extra_workloads`: the other benchmark configurations (64k tokens at T=0.7, the Qwen3 head in
    f16 with 1 % ignored positions, the GRPO step with its loss epilogue, the logits-fed scan) and
    the shapes the reference publishes H100 latencies for, fp32 inputs, a few steps each;
  * `cpu_baseline`: the CPU oracle (F.linear -> log_softmax -> gather in fp32, autograd backward)
    timed on a 2048-token slice on the host cores.
"""

from __future__ import annotations

import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0}  # MI355X dense MFMA, published
PEAK_HBM_GBS = 8000.0

# HBM-side bytes moved by ONE launch of each kernel at the default workload, from two
# `rocprofv3 --pmc` runs of this script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled
# by what the same counter reads for the 1 GiB `--calibrate-copy` kernel.  The figures belong to
# the kernel sources whose digest is recorded with them; with other sources `traffic` is null.
MEASURED_TRAFFIC = {
    "workload": "llama3-8b-head",
    "kernel_source_sha16": "27f6927cb1dd4afa",
    "measured_at_commit": "ed6874b",
    "counter_scale": {"FETCH_SIZE": 2.000, "WRITE_SIZE": 1.000},
    "bytes_per_launch": {
        "linear_logp_fwd_kernel": 57634103170,
        "linear_logp_dz_kernel": 1958119534,
        "linear_logp_dh_kernel": 1834437792,
        "linear_logp_dw_kernel": 2108737019,
    },
}

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
    # fp32 hidden states and head on the fp32 matrix instruction (two shapes, see bench_fp32_inputs)
    "fp32-inputs": dict(tokens=4096, hidden=2048, vocab=32768, dtype="f32", temperature=1.0,
                        ignore_frac=0.0, fp32=True),
}

# linear_logp latencies the reference publishes (docs/operators/linear-logp.md:116-132 of the
# reference: NVIDIA H100 80GB, bf16, N=4096, D=2048), in ms: forward, forward+backward
REFERENCE_PUBLISHED_H100 = {
    32768: {"fwd_ms": {"native": 1.79, "triton": 6.42, "sm90": 3.41},
            "fwd_bwd_ms": {"native": 4.25, "triton": 15.86, "sm90": 12.69}},
    50257: {"fwd_ms": {"native": 9.96, "triton": 9.82, "sm90": 4.88},
            "fwd_bwd_ms": {"native": 23.29, "triton": 47.20, "sm90": 42.20}},
    131072: {"fwd_ms": {"native": 7.28, "triton": 25.56, "sm90": 12.88},
             "fwd_bwd_ms": {"native": 17.05, "triton": 117.62, "sm90": 104.97}},
}


KERNEL_SOURCES = ("rlk_common.hpp", "rlk_gemm.hpp", "rlk_grpo.hpp", "rlk_linear_logp.hip",
                  "rlk_tile_epilogue.hpp")


def kernel_source_sha16() -> str:
    """Digest of the sources the four contraction kernels are compiled from (the file that holds
    them and the headers it includes)."""
    m = hashlib.sha256()
    csrc = os.path.join(ROOT, "rl-kernel_amd", "csrc")
    for name in KERNEL_SOURCES:
        with open(os.path.join(csrc, name), "rb") as fh:
            m.update(name.encode())
            m.update(fh.read())
    return m.hexdigest()[:16]


def make_inputs(torch, cfg, device, seed=1002):
    """hidden ~ N(0,1), weight ~ N(0, 0.02^2), targets uniform (a Bernoulli(ignore_frac) share set
    to -100), upstream gradient ~ N(0,1), from the counter-based generator: every value is a function
    of (seed, tensor id, element index) in integer arithmetic, so the inputs do not depend on the
    device or on the torch / rocRAND build (tensor ids: 0 hidden, 1 weight, 2 targets, 3 ignored
    positions, 4 upstream gradient)."""
    from rl_kernel_amd import synthetic as S

    dt = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float16
    n, h, v = cfg["tokens"], cfg["hidden"], cfg["vocab"]
    hidden = S.normal(seed, 0, (n, h), dtype=dt, device=device)
    weight = S.normal(seed, 1, (v, h), std=0.02, dtype=dt, device=device)
    targets = S.randint(seed, 2, (n,), v, device=device)
    if cfg["ignore_frac"] > 0:
        drop = S.bernoulli(seed, 3, (n,), cfg["ignore_frac"], device=device)
        targets = torch.where(drop, torch.full_like(targets, -100), targets)
    grad = S.normal(seed, 4, (n,), device=device)
    return hidden, weight, targets, grad


def cpu_baseline(torch, cfg, slice_tokens, iters=2):
    """Time the CPU oracle on a token slice: fp32 F.linear -> log_softmax -> gather forward, torch
    autograd backward (what the reference's CPU path does for a training step)."""
    from oracle import oracle as O

    gen = torch.Generator().manual_seed(7)
    h, v = cfg["hidden"], cfg["vocab"]
    hidden = torch.randn(slice_tokens, h, generator=gen).requires_grad_(True)
    weight = (torch.randn(v, h, generator=gen) * 0.02).requires_grad_(True)
    targets = torch.randint(0, v, (slice_tokens,), generator=gen)
    grad = torch.randn(slice_tokens, generator=gen)

    def step():
        hidden.grad = None
        weight.grad = None
        logp = O.linear_logp(hidden, weight, targets, temperature=cfg["temperature"])
        logp.backward(grad)

    step()  # warm-up
    times = []
    for _ in range(iters):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2] if len(times) % 2 else 0.5 * (times[len(times) // 2 - 1] + times[len(times) // 2])
    return {
        "value": slice_tokens / med,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{slice_tokens}-token slice at the full H={h}, V={v}; fp32 torch CPU oracle "
                  f"(F.linear -> log_softmax -> gather) forward + autograd backward, 1 warm-up + "
                  f"{iters} timed, median; host cpu_count={os.cpu_count()}",
    }


def device_info(torch):
    """Name, compute units and maximum engine clock as the HIP runtime reports them, and the 16-bit
    matrix-core peak they imply (CU x 4096 flop per clock x clock) next to the published one."""
    import ctypes

    from rl_kernel_amd import _native

    p = torch.cuda.get_device_properties(0)
    info = {"name": p.name, "compute_units": p.multi_processor_count}
    cu, khz = ctypes.c_int32(0), ctypes.c_int32(0)
    if _native.load().rlk_device_info(0, ctypes.byref(cu), ctypes.byref(khz)) == 0 and khz.value > 0:
        info["compute_units"] = cu.value
        info["max_sclk_mhz"] = khz.value / 1e3
        info["peak_from_cu_clock_tflops"] = cu.value * 4096 * khz.value * 1e3 / 1e12
        info["published_peak_tflops"] = PEAK_TFLOPS["bf16"]
    return info


def event_ms(torch, fn, reps):
    """Average duration of fn() over `reps` back-to-back calls, by HIP events on the current
    stream (the stream every kernel of this library is launched on)."""
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def bench_scan(torch, steps, warmup, cfg):
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
    for _ in range(warmup):
        logp_from_logits(logits, ids, out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    k_ms = event_ms(torch, lambda: logp_from_logits(logits, ids, out), steps)
    ms = (time.perf_counter() - t0) * 1e3 / steps
    nbytes = float(n * v * logits.element_size() + n * 8 + n * 4)
    return {
        "metric": "logp from logits tokens/sec", "value": n / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": f"logits-scan: selected-token logp from {n} x {v} {cfg['dtype']} logits",
                   "tokens": n, "vocab": v},
        "bitwise_repeatable": bool(torch.equal(first, out)),
        "roofline": {"kernel": "logp_scan_kernel", "bound": "hbm", "achieved": nbytes / (k_ms * 1e-3) / 1e9,
                     "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": nbytes / (k_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                     "traffic": None, "algorithmic_bytes": nbytes, "launch_ms": k_ms},
    }


def bwd_plan(n, h, v, dtype_id):
    import ctypes

    from rl_kernel_amd import _native

    out = (ctypes.c_int64 * 5)()
    _native.check(_native.load().rlk_linear_logp_bwd_plan(n, h, v, dtype_id, 0, out), "plan")
    return dict(tok_chunk=out[0], v_piece=out[1], n_chunks=out[2], n_pieces=out[3], dh_parts=out[4])


def fwd_plan(n, h, v, dtype_id):
    import ctypes

    from rl_kernel_amd import _native

    out = (ctypes.c_int64 * 4)()
    _native.check(_native.load().rlk_linear_logp_fwd_plan(n, h, v, dtype_id, out), "plan")
    wgs = out[0] * out[1]
    return dict(token_blocks=out[0], vocab_splits=out[1], ragged_tile_splits=out[2],
                token_blocks_per_xcd_patch=out[3], workgroups=wgs, rounds_of_256_cus=wgs / 256.0)


def bench_linear(torch, name, cfg, steps, warmup, mode="fwd+bwd", detailed=False, registry_op=False,
                 probe_epilogue=True, kernel_timing=True):
    """Forward(+backward) of the fused LM-head logp through the raw C-ABI wrappers."""
    from rl_kernel_amd.ops import linear_logp as LL

    dev = torch.device("cuda:0")
    hidden, weight, targets, grad = make_inputs(torch, cfg, dev)
    n, h, v = cfg["tokens"], cfg["hidden"], cfg["vocab"]
    ign = -100 if cfg["ignore_frac"] > 0 else None
    temp = cfg["temperature"]
    do_bwd = mode == "fwd+bwd"
    peak = PEAK_TFLOPS[cfg["dtype"]]
    grpo = cfg.get("grpo")
    if grpo:
        from rl_kernel_amd.ops import grpo as GR
        from rl_kernel_amd.ops import grpo_step as GS

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

    def forward():
        return LL.fused_linear_logp_forward(hidden, weight, targets, None, temperature=temp,
                                            ignore_index=ign)

    def backward(upstream, lse, need_hidden=True, need_weight=True):
        return LL.fused_linear_logp_backward(upstream, hidden, weight, targets, lse, None,
                                             temperature=temp, ignore_index=ign,
                                             need_hidden=need_hidden, need_weight=need_weight)

    def grpo_forward():
        # group advantages, then the forward whose last launch emits the loss terms and d loss / d logp
        adv = GR.group_advantages(rewards, samples_per_prompt=g)
        return GS.fused_linear_logp_grpo_forward(hidden, weight, targets, None, old, ref, adv, mask,
                                                 seq_len=t, clip_eps=grpo["clip_eps"],
                                                 beta=grpo["beta"], temperature=temp, ignore_index=ign)

    def step(record=False):
        if grpo:
            logp, lse, _, out3, _, _, d_cur, _ = grpo_forward()
            d_h, d_w, _ = backward(d_cur, lse)
            return (logp, lse, out3, d_h, d_w)
        logp, lse, _ = forward()
        if not do_bwd:
            return (logp, lse)
        d_h, d_w, _ = backward(grad, lse)
        return (logp, lse, d_h, d_w)

    torch.cuda.synchronize()
    base_mem = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    first = step()
    torch.cuda.synchronize()
    out_bytes = sum(t.numel() * t.element_size() for t in first)
    peak_extra = torch.cuda.max_memory_allocated() - base_mem - out_bytes
    for _ in range(max(0, warmup - 1)):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    last = None
    for _ in range(steps):
        last = step(record=True)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    deterministic = all(torch.equal(a, b) for a, b in zip(first, last))
    lse = last[1]
    del first, last

    step_flops = (8.0 if do_bwd else 2.0) * n * h * v
    res = {
        "metric": "logp fwd+bwd tokens/sec" if do_bwd else "logp fwd tokens/sec",
        "value": n / (ms * 1e-3),
        "unit": "tokens/s",
        "ms_per_step": ms,
        "dtype": cfg["dtype"],
        "config": {
            "workload": f"{name}: fused LM-head logp {mode}, {n} tokens, H={h}, "
                        f"V={v}, {cfg['dtype']} in / fp32 accumulate, T={temp}",
            "tokens": n, "hidden": h, "vocab": v, "mode": mode,
        },
        "step_tflops": step_flops / (ms * 1e-3) / 1e12,
        "step_frac_of_mfma_peak": step_flops / (ms * 1e-3) / 1e12 / peak,
        "step_flop_accounting": "8*N*H*V (fwd 2 + logit recompute 2 + dH 2 + dW 2)" if do_bwd
                                else "2*N*H*V",
        "step_tflops_no_recompute_accounting": (6.0 if do_bwd else 2.0) * n * h * v / (ms * 1e-3) / 1e12,
        "peak_extra_hbm_bytes": int(peak_extra),
        "peak_extra_hbm_note": "raw C ABI: logp, lse, dH and the fp32 dW are declared outputs; what "
                               "is counted is workspace (split partials, one dZ block, fp32 dH chunk)",
        "bitwise_repeatable": bool(deterministic),
    }
    if grpo:
        res["metric"] = "GRPO step (logp fwd + loss epilogue + bwd) tokens/sec"
    if grpo and probe_epilogue:
        # The loss epilogue rides in the forward's last launch.  At the full head its cost drowns
        # in the +-1 % run-to-run spread of the 25 ms contraction, so it is measured where the
        # contraction is negligible: the same 32768 tokens, masks, advantages and log-prob inputs
        # on a tiny head (H=64, V=512), forward with epilogue minus plain forward.
        plain = event_ms(torch, forward, 5)
        fused = event_ms(torch, grpo_forward, 5)
        th = torch.randn(n, 64, device=dev).to(hidden.dtype)
        tw = (torch.randn(512, 64, device=dev) * 0.1).to(hidden.dtype)
        tt = torch.where(mask.reshape(-1), targets % 512, torch.full_like(targets, -100))
        adv0 = GR.group_advantages(rewards, samples_per_prompt=g)

        def tiny_plain():
            return LL.fused_linear_logp_forward(th, tw, tt, None, temperature=temp, ignore_index=ign)

        def tiny_fused():
            adv = GR.group_advantages(rewards, samples_per_prompt=g)
            return GS.fused_linear_logp_grpo_forward(th, tw, tt, None, old, ref, adv, mask, seq_len=t,
                                                     clip_eps=grpo["clip_eps"], beta=grpo["beta"],
                                                     temperature=temp, ignore_index=ign)

        def two_step_epilogue():
            adv = GR.group_advantages(rewards, samples_per_prompt=g)
            return GR.grpo_from_logp_raw(lse.view(g, t), old, ref, adv, mask, clip_eps=grpo["clip_eps"],
                                         beta=grpo["beta"], want_grad=True)

        def graph_ms(fn, replays=200):
            # the launches of fn() recorded once into a HIP graph and replayed: device time
            # without the host's launch gaps
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                keep = fn()
            graph.replay()
            ms_ = event_ms(torch, graph.replay, replays)
            del keep, graph
            return ms_

        tiny_p = graph_ms(tiny_plain)
        tiny_f = graph_ms(tiny_fused)
        two_step = graph_ms(two_step_epilogue)
        epi_ms = max(tiny_f - tiny_p, 1e-4)
        del th, tw, tt, adv0
        epi_bytes = n * (4 + 4 + 4 + 1 + 4 + 4)  # cur, old, ref, mask in; d_cur, d_kl out
        res["epilogue"] = {
            "bound": "hbm", "ms": epi_ms, "algorithmic_bytes": epi_bytes,
            "full_head_forward_ms": plain, "full_head_forward_with_epilogue_ms": fused,
            "tiny_head_forward_ms": tiny_p, "tiny_head_forward_with_epilogue_ms": tiny_f,
            "stand_alone_epilogue_ms": two_step,
            "achieved": epi_bytes / (epi_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": epi_bytes / (epi_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
            "note": "group advantages + active-token count + loss terms, gradient and the final sums "
                    "inside the launch that merges the vocab splits; ms = forward with "
                    "epilogue minus plain forward on a tiny head with the same tokens, each recorded "
                    "into a HIP graph and replayed 200 times (device time, no host launch gaps); "
                    "stand_alone_epilogue_ms = the same math as separate launches on ready "
                    "log-probs, measured the same way; 0.7 MB of traffic: launch-latency-bound",
            "active_tokens": int(mask.sum().item()),
        }

    if grpo and kernel_timing:
        res["skip_masked"] = bench_skip_masked(torch, hidden, weight, targets, mask, old, ref, rewards,
                                               grpo, temp, max(3, steps // 2))

    # per-kernel launch times by HIP events: the forward on its own; the three backward kernels
    # from backward calls with one gradient switched off (dZ+dH, dZ+dW, all three), by difference
    if not kernel_timing:
        # a profiler run reads the launch times from the kernel trace: keep its call counts at
        # steps x launches per step
        res["kernel_source_sha16"] = kernel_source_sha16()
        return res
    reps = 3 if detailed else 2
    fwd_ms = event_ms(torch, forward, reps)
    fwd_flops = 2.0 * n * h * v
    kernels = [{"kernel": "linear_logp_fwd_kernel", "launches_per_step": 1, "launch_ms": fwd_ms,
                "flops_per_launch": fwd_flops, "achieved": fwd_flops / (fwd_ms * 1e-3) / 1e12,
                "algorithmic_bytes": float((n * h + v * h) * 2 + n * 8 + n * 8)}]
    if do_bwd and detailed:
        plan = bwd_plan(n, h, v, 0 if cfg["dtype"] == "bf16" else 1)
        blocks = plan["n_chunks"] * plan["n_pieces"]
        t_all = event_ms(torch, lambda: backward(grad, lse), reps)
        t_h = event_ms(torch, lambda: backward(grad, lse, need_weight=False), reps)
        t_w = event_ms(torch, lambda: backward(grad, lse, need_hidden=False), reps)
        blk_flops = 2.0 * n * h * v / blocks
        elt = 2
        c, p = min(plan["tok_chunk"], n), min(plan["v_piece"], v)
        alg = {"linear_logp_dz_kernel": (c * h + p * h + c * p) * elt,
               "linear_logp_dh_kernel": (c * p + p * h) * elt + c * h * 4,
               "linear_logp_dw_kernel": (c * p + c * h) * elt + p * h * 4}
        for kname, total in (("linear_logp_dz_kernel", t_h + t_w - t_all),
                             ("linear_logp_dh_kernel", t_all - t_w),
                             ("linear_logp_dw_kernel", t_all - t_h)):
            kernels.append({"kernel": kname, "launches_per_step": blocks,
                            "launch_ms": total / blocks, "flops_per_launch": blk_flops,
                            "achieved": blk_flops / (total / blocks * 1e-3) / 1e12,
                            "algorithmic_bytes": float(alg[kname])})
        res["backward_plan"] = plan
        res["forward_plan"] = fwd_plan(n, h, v, 0 if cfg["dtype"] == "bf16" else 1)
        res["backward_ms"] = t_all
        res["kernel_timing_method"] = (
            "HIP events on the launch stream; forward alone; backward kernels from three backward "
            "calls (all gradients, without dW, without dH) by difference, divided by the number of "
            "(token chunk x vocab piece) blocks")
    sha = kernel_source_sha16()
    for k in kernels:
        k.update({"bound": "mfma", "peak": peak, "unit": "TFLOP/s", "frac": k["achieved"] / peak})
        traffic = None
        if name == MEASURED_TRAFFIC["workload"] and sha == MEASURED_TRAFFIC["kernel_source_sha16"]:
            traffic = MEASURED_TRAFFIC["bytes_per_launch"].get(k["kernel"])
        k["traffic"] = traffic
    if name == MEASURED_TRAFFIC["workload"]:
        res["traffic_source"] = (
            f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE at commit {MEASURED_TRAFFIC['measured_at_commit']} "
            f"(kernel sources {MEASURED_TRAFFIC['kernel_source_sha16']}), see profiles/"
            if sha == MEASURED_TRAFFIC["kernel_source_sha16"] else
            f"null: the kernel sources ({sha}) differ from the ones the counters were read with "
            f"({MEASURED_TRAFFIC['kernel_source_sha16']})")
    res["kernels"] = kernels
    res["kernel_source_sha16"] = sha
    dominant = max(kernels, key=lambda k: k["launch_ms"] * k["launches_per_step"])
    res["roofline"] = dict(dominant)
    res["roofline"]["note"] = "the kernel with the largest share of the step; see `kernels` for all four"

    if registry_op and do_bwd and not grpo:
        res["through_registry_op"] = bench_registry_op(torch, hidden, weight, targets, grad, temp, ign,
                                                       max(3, steps // 2))
    return res


def bench_skip_masked(torch, hidden, weight, targets, mask, old, ref, rewards, grpo, temp, steps):
    """The GRPO step through the caller-side glue (`training.grpo_loss_step`, autograd), once with
    every position carried through the kernels and once with the masked positions taken out
    (`skip_masked`): the same values to fp32 rounding; the work shrinks by the masked share."""
    from rl_kernel_amd.training import grpo_loss_step

    g, t = grpo["group"], grpo["seq"]
    head = torch.nn.Linear(1, 1, bias=False)
    head.in_features, head.out_features = weight.shape[1], weight.shape[0]
    head.weight = torch.nn.Parameter(weight)  # shares the storage
    hid = hidden.view(g, t, -1).detach().requires_grad_(True)
    ids = torch.where(mask, targets.view(g, t), torch.zeros_like(targets.view(g, t)))
    out = {"active_tokens": int(mask.sum().item()), "tokens": int(mask.numel())}
    keep = {}
    for key, skip in (("all_positions_ms", False), ("skip_masked_ms", True)):
        def step():
            hid.grad = None
            head.weight.grad = None
            r = grpo_loss_step(hid, head, ids, mask, old, ref, rewards, samples_per_prompt=g,
                               clip_eps=grpo["clip_eps"], beta=grpo["beta"], temperature=temp,
                               skip_masked=skip)
            r.loss.backward()
            return r
        step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            r = step()
        torch.cuda.synchronize()
        out[key] = (time.perf_counter() - t0) * 1e3 / steps
        keep[key] = (r.loss.detach().clone(), r.current_logps.detach().clone(), hid.grad.clone())
    a, b = keep["all_positions_ms"], keep["skip_masked_ms"]
    rel = lambda x, y: float((x.float() - y.float()).norm() / y.float().norm())
    out["difference"] = {"loss_abs": abs(float(a[0]) - float(b[0])),
                         "logp_max_abs": float((a[1] - b[1]).abs().max()),
                         "dH_rel_norm": rel(b[2], a[2])}
    out["note"] = ("wall clock per step through autograd, bf16 dW returned (the fp32 dW is cast); "
                   "skip_masked gathers the unmasked rows, runs the head's kernels on them and puts "
                   "the results back; tokens/s of the headline counts every position as computed "
                   "and is NOT taken from this mode")
    head.weight.grad = None
    return out


def bench_registry_op(torch, hidden, weight, targets, grad, temp, ign, steps):
    """The same step through kernel_registry.get_op('linear_logp') and autograd."""
    from rl_kernel_amd.registry import kernel_registry

    op = kernel_registry.get_op("linear_logp")
    hid = hidden.detach().requires_grad_(True)
    w = weight.detach().requires_grad_(True)

    def step():
        hid.grad = None
        w.grad = None
        out = op(hid, w, targets, temperature=temp, ignore_index=ign)
        out.backward(grad)
        return out

    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    out = step()
    torch.cuda.synchronize()
    declared = out.numel() * 4 + hid.grad.numel() * hid.grad.element_size() + \
        w.grad.numel() * w.grad.element_size()
    peak_extra = torch.cuda.max_memory_allocated() - base - declared
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    n = hidden.size(0)
    res = {"class": type(op).__name__, "ms_per_step": ms, "tokens_per_s": n / (ms * 1e-3),
           "steps": steps, "peak_extra_hbm_bytes": int(peak_extra),
           "note": "declared outputs here are logp, dH and dW in the weight dtype; the extra bytes "
                   "include the fp32 dW the kernels accumulate into before the cast (as the "
                   "reference's backward keeps an fp32 grad_w) and the saved lse"}
    del out
    hid.grad = None
    w.grad = None
    torch.cuda.empty_cache()

    # the same step with the weight gradient added into the caller's fp32 buffer (main gradients):
    # no [V, H] temporary, no cast; the target check reads a device flag (check_targets=False skips
    # the host synchronisation the reference's ValueError convention costs)
    main_grad = torch.zeros(weight.shape, device=weight.device, dtype=torch.float32)

    def step_main():
        hid.grad = None
        out = op(hid, w, targets, temperature=temp, ignore_index=ign, weight_grad_out=main_grad,
                 check_targets=False)
        out.backward(grad)
        return out

    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    out = step_main()
    torch.cuda.synchronize()
    declared = out.numel() * 4 + hid.grad.numel() * hid.grad.element_size()
    peak_main = torch.cuda.max_memory_allocated() - base - declared
    t0 = time.perf_counter()
    for _ in range(steps):
        step_main()
    torch.cuda.synchronize()
    ms_main = (time.perf_counter() - t0) * 1e3 / steps
    res["into_main_grad"] = {
        "ms_per_step": ms_main, "tokens_per_s": n / (ms_main * 1e-3), "steps": steps,
        "peak_extra_hbm_bytes": int(peak_main),
        "note": "op(..., weight_grad_out=<fp32 [V,H] buffer of the caller>, check_targets=False): the "
                "backward adds dW into the buffer (rlk_linear_logp_bwd_accum); declared outputs are "
                "logp and dH; extra bytes = workspace + saved lse"}
    return res


def window_ms(torch, fn, min_ms, min_calls=4, idle_s=0.0):
    """fn() back to back for at least `min_ms` of device time: (ms per call, calls, total ms)."""
    fn()
    one = event_ms(torch, fn, 1)
    calls = max(min_calls, int(min_ms / max(one, 1e-3)) + 1)
    if idle_s:
        time.sleep(idle_s)
    total = event_ms(torch, fn, calls) * calls
    return total / calls, calls, total


def bench_library_gemm(torch, cfg):
    """Vendor GEMM (torch.matmul -> hipBLASLt) on the same box, same operands, for scale: the work of
    one forward (8 GEMMs [N,H] x [H,V/8] into one reused output; the library writes the logits it
    computes) sustained over >= 150 ms, the same as a burst after an idle period, the shapes of one
    dH and one dW block, and the fused forward / backward over windows of the same length."""
    from rl_kernel_amd.ops import linear_logp as LL

    dev = torch.device("cuda:0")
    hidden, weight, targets, grad = make_inputs(torch, cfg, dev)
    n, h, v = cfg["tokens"], cfg["hidden"], cfg["vocab"]
    piece = v // 8
    pieces = [weight[i * piece:(i + 1) * piece] for i in range(8)]
    out = torch.empty(n, piece, device=dev, dtype=hidden.dtype)
    flop = 2.0 * n * h * piece * 8

    def lib_forward():
        for p in pieces:
            torch.matmul(hidden, p.t(), out=out)

    def tf(f, ms):
        return f / (ms * 1e-3) / 1e12

    res = {"what": f"torch.matmul (hipBLASLt), {cfg['dtype']}: 8 x [{n},{h}] x [{h},{piece}] = the "
                   "contraction work of one forward, output reused; TFLOP/s with the window they "
                   "were measured over"}
    ms, calls, total = window_ms(torch, lib_forward, 150.0)
    res["sustained_tflops"] = tf(flop, ms)
    res["sustained_window_ms"] = total
    ms_b, _, total_b = window_ms(torch, lib_forward, 1.0, min_calls=1, idle_s=1.0)
    res["burst_tflops"] = tf(flop, ms_b)
    res["burst_window_ms"] = total_b
    res["burst_note"] = "one pass of the 8 GEMMs after 1 s of idle (clocks ramp up from idle)"
    ms_f, _, total_f = window_ms(torch, lambda: LL.fused_linear_logp_forward(hidden, weight, targets), 150.0)
    res["fused_forward_sustained_tflops"] = tf(2.0 * n * h * v, ms_f)
    res["fused_forward_window_ms"] = total_f
    # block shapes of the backward: dH = dZ [c,p] x W [p,h] (NN), dW = dZ^T [p,c] x H [c,h] (TN)
    c, p = min(8192, n), min(16384, v)
    dz = (torch.randn(c, p, device=dev) * 0.01).to(hidden.dtype)
    w_p, h_c = weight[:p], hidden[:c]
    o_h = torch.empty(c, h, device=dev, dtype=hidden.dtype)
    o_w = torch.empty(p, h, device=dev, dtype=hidden.dtype)
    blk = 2.0 * c * p * h
    ms_h, _, tot_h = window_ms(torch, lambda: torch.matmul(dz, w_p, out=o_h), 100.0)
    ms_w, _, tot_w = window_ms(torch, lambda: torch.matmul(dz.t(), h_c, out=o_w), 100.0)
    res["dh_block_shape_nn_sustained_tflops"] = tf(blk, ms_h)
    res["dw_block_shape_tn_sustained_tflops"] = tf(blk, ms_w)
    res["block_shape"] = f"dZ [{c},{p}], 16-bit output (the fused kernels accumulate dW in fp32)"
    _, lse, _ = LL.fused_linear_logp_forward(hidden, weight, targets)
    ms_bw, _, tot_bw = window_ms(torch, lambda: LL.fused_linear_logp_backward(grad, hidden, weight, targets, lse),
                                 150.0, min_calls=2)
    res["fused_backward_sustained_tflops"] = tf(6.0 * n * h * v, ms_bw)
    res["fused_backward_window_ms"] = tot_bw
    return res


def bench_variants(torch, cfg):
    """The caller-side variants of the head at the default shape: final RMSNorm inside the call
    (forward and backward take the un-normalised hidden states) and policy + reference head in one
    forward launch, each next to the plain call, HIP events, 3 calls each."""
    from rl_kernel_amd.ops import linear_logp as LL

    dev = torch.device("cuda:0")
    hidden, weight, targets, grad = make_inputs(torch, cfg, dev)
    n, h, v = cfg["tokens"], cfg["hidden"], cfg["vocab"]
    gain = (1.0 + 0.1 * torch.randn(h, device=dev)).to(hidden.dtype)
    ref_weight = (weight.float() * 1.01).to(weight.dtype)
    _, lse, _ = LL.fused_linear_logp_forward(hidden, weight, targets)
    _, lse_n, _ = LL.fused_norm_linear_logp_forward(hidden, gain, weight, targets)
    out = {
        "forward_ms": event_ms(torch, lambda: LL.fused_linear_logp_forward(hidden, weight, targets), 3),
        "forward_with_rmsnorm_ms": event_ms(
            torch, lambda: LL.fused_norm_linear_logp_forward(hidden, gain, weight, targets), 3),
        "forward_two_heads_ms": event_ms(
            torch, lambda: LL.fused_linear_logp_forward_pair(hidden, weight, ref_weight, targets), 3),
        "backward_ms": event_ms(
            torch, lambda: LL.fused_linear_logp_backward(grad, hidden, weight, targets, lse), 3),
        "backward_with_rmsnorm_ms": event_ms(
            torch, lambda: LL.fused_norm_linear_logp_backward(grad, hidden, gain, weight, targets, lse_n), 3),
        "note": f"{n} tokens, H={h}, V={v}, {cfg['dtype']}; with_rmsnorm: the call takes the "
                "un-normalised hidden states and the norm gain (normalised rows only in workspace, "
                "d_x and d_gain returned); two_heads: policy and reference head in one launch "
                "(twice the contraction work of forward_ms)",
    }
    return out


def bench_reference_shapes(torch):
    """The reference's own benchmark shapes and method (benchmarks/benchmark_linear_logp.py:62-86:
    bf16, hidden ~ N(0,1), weight ~ N(0,1), warm-up 5, 20 iterations between device events),
    through the op class and autograd, next to the H100 latencies the reference publishes."""
    from rl_kernel_amd.registry import kernel_registry

    op = kernel_registry.get_op("linear_logp")
    dev = torch.device("cuda:0")
    rows = []
    for vocab, published in REFERENCE_PUBLISHED_H100.items():
        n, d = 4096, 2048
        gen = torch.Generator(device=dev).manual_seed(vocab)
        hidden = torch.randn(n, d, device=dev, generator=gen).to(torch.bfloat16).requires_grad_(True)
        weight = torch.randn(vocab, d, device=dev, generator=gen).to(torch.bfloat16).requires_grad_(True)
        target = torch.randint(0, vocab, (n,), device=dev, generator=gen)

        def fwd():
            with torch.no_grad():
                return op(hidden, weight, target)

        def fwd_bwd():
            hidden.grad = None
            weight.grad = None
            op(hidden, weight, target).sum().backward()

        for _ in range(5):
            fwd()
            fwd_bwd()
        rows.append({"shape": f"{n}x{d}x{vocab}", "fwd_ms": event_ms(torch, fwd, 20),
                     "fwd_bwd_ms": event_ms(torch, fwd_bwd, 20),
                     "reference_h100_ms": published})
        del hidden, weight
    return {"what": "linear_logp latency at the shapes of the reference's published table, op class + "
                    "autograd on one MI355X; reference_h100_ms are the reference's own H100 figures "
                    "(other hardware: context, not a like-for-like baseline)",
            "rows": rows}


def bench_fp32_inputs(torch):
    """fp32 hidden states and head (what the reference runs in its CPU tests and what callers that keep
    an fp32 lm_head pass): the same entry points on the fp32 matrix instruction, priced against the
    157.3 TFLOP/s fp32 matrix peak; a plain fp32 library GEMM of the forward's shape beside it."""
    from rl_kernel_amd.ops import linear_logp as LL

    dev = torch.device("cuda:0")
    rows = []
    for n, h, v in ((4096, 2048, 32768), (2048, 4096, 128256)):
        gen = torch.Generator(device=dev).manual_seed(v)
        hidden = torch.randn(n, h, device=dev, generator=gen)
        weight = torch.randn(v, h, device=dev, generator=gen) * 0.02
        target = torch.randint(0, v, (n,), device=dev, generator=gen)
        grad = torch.randn(n, device=dev, generator=gen)
        _, lse, _ = LL.fused_linear_logp_forward(hidden, weight, target)
        fwd = lambda: LL.fused_linear_logp_forward(hidden, weight, target)
        bwd = lambda: LL.fused_linear_logp_backward(grad, hidden, weight, target, lse)
        gemm = lambda: torch.matmul(hidden, weight.t())
        for f in (fwd, bwd, gemm):
            f()
        f_ms, b_ms, g_ms = event_ms(torch, fwd, 5), event_ms(torch, bwd, 3), event_ms(torch, gemm, 5)
        flop = 2.0 * n * h * v
        rows.append({"shape": f"{n}x{h}x{v}", "fwd_ms": f_ms, "bwd_ms": b_ms,
                     "fwd_tflops": flop / f_ms / 1e9, "bwd_tflops": 3.0 * flop / b_ms / 1e9,
                     "fwd_frac_of_fp32_peak": flop / f_ms / 1e9 / 157.3,
                     "bwd_frac_of_fp32_peak": 3.0 * flop / b_ms / 1e9 / 157.3,
                     "library_fp32_gemm_tflops": flop / g_ms / 1e9})
        del hidden, weight
    return {"what": "rlk_linear_logp_fwd / _bwd on fp32 inputs (v_mfma_f32_32x32x2_f32 tiles), "
                    "TFLOP/s on 2NHV / 6NHV, peak 157.3 TFLOP/s", "rows": rows}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama3-8b-head", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-slice", type=int, default=2048,
                    help="tokens of the CPU-baseline slice (0 = skip the CPU baseline)")
    ap.add_argument("--mode", default="fwd+bwd", choices=["fwd+bwd", "fwd"])
    ap.add_argument("--dtype", default=None, choices=["bf16", "f16"],
                    help="override the workload's 16-bit input type")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the extra workloads, the registry-op timing, the vendor GEMM and the "
                         "tiny-head probe of the loss epilogue (what a profiler run wants)")
    ap.add_argument("--no-kernel-timing", action="store_true",
                    help="skip the per-kernel launch timing (extra forward / backward calls after the "
                         "timed steps): under rocprofv3 the kernel trace then holds exactly "
                         "(warmup + steps) x launches per step")
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

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cfg = dict(WORKLOADS[args.workload])
    if args.dtype:
        cfg["dtype"] = args.dtype
    common = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True,
              "scaling": "weak", "vs_baseline": None, "data": "synthetic", "seed": 1002,
              "input_generator": "counter-based: splitmix64(seed, tensor id, index) -> Irwin-Hall normal / "
                                 "uniform index in integer arithmetic (rl-kernel_amd/synthetic.py), the same "
                                 "bits on CPU and GPU"}

    if args.calibrate_copy:
        src = torch.ones(1 << 28, device=dev, dtype=torch.float32)   # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        torch.neg(src, out=dst)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    if cfg.get("scan"):
        result = bench_scan(torch, args.steps, args.warmup, cfg)
        result["device"] = device_info(torch)
        print(json.dumps(result))
        return 0

    if cfg.get("fp32"):
        r = bench_fp32_inputs(torch)
        row = r["rows"][0]
        result = dict(common)
        result.update({"metric": "linear_logp tokens/s (fwd+bwd)", "unit": "tokens/s", "dtype": "f32",
                       "value": 4096 / ((row["fwd_ms"] + row["bwd_ms"]) * 1e-3),
                       "ms_per_step": row["fwd_ms"] + row["bwd_ms"],
                       "config": {"workload": "fp32-inputs: " + row["shape"] + " fp32, fwd + bwd"},
                       "fp32": r, "device": device_info(torch)})
        print(json.dumps(result))
        return 0

    main_default = args.workload == "llama3-8b-head" and args.mode == "fwd+bwd" and not args.no_extras
    result = dict(common)
    result.update(bench_linear(torch, args.workload, cfg, args.steps, args.warmup, args.mode,
                               detailed=True, registry_op=not args.no_extras,
                               probe_epilogue=not args.no_extras,
                               kernel_timing=not args.no_kernel_timing))
    result["device"] = device_info(torch)
    torch.cuda.empty_cache()

    if not args.no_extras:
        try:
            result["library_gemm"] = bench_library_gemm(torch, cfg)
        except Exception as exc:  # the comparison is optional
            result["library_gemm"] = {"error": str(exc)[:200]}
        torch.cuda.empty_cache()

    if main_default:
        extras = {}
        for name in ("llama3-8b-head-64k", "qwen3-head", "llama3-8b-grpo-step"):
            r = bench_linear(torch, name, dict(WORKLOADS[name]), 3, 1, "fwd+bwd", detailed=False)
            keep = ("metric", "value", "unit", "ms_per_step", "dtype", "config", "step_tflops",
                    "step_frac_of_mfma_peak", "peak_extra_hbm_bytes", "bitwise_repeatable",
                    "epilogue", "skip_masked")
            extras[name] = {k: r[k] for k in keep if k in r}
            extras[name]["forward_launch_ms"] = r["kernels"][0]["launch_ms"]
            extras[name]["forward_tflops"] = r["kernels"][0]["achieved"]
            extras[name]["steps"] = 3
            torch.cuda.empty_cache()
        extras["llama3-8b-head-variants"] = bench_variants(torch, dict(WORKLOADS["llama3-8b-head"]))
        torch.cuda.empty_cache()
        r = bench_scan(torch, 10, 2, dict(WORKLOADS["logits-scan"]))
        extras["logits-scan"] = {k: r[k] for k in ("metric", "value", "unit", "ms_per_step", "config",
                                                   "bitwise_repeatable", "roofline")}
        torch.cuda.empty_cache()
        extras["reference-published-shapes"] = bench_reference_shapes(torch)
        extras["fp32-inputs"] = bench_fp32_inputs(torch)
        torch.cuda.empty_cache()
        result["extra_workloads"] = extras

    if args.cpu_slice > 0:
        result["cpu_baseline"] = cpu_baseline(torch, cfg, args.cpu_slice)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
