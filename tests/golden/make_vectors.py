#!/usr/bin/env python3
"""Writes tests/golden/seeded_vectors.npz: seeded inputs of the fused log-prob path and the outputs
the double-precision C oracle (oracle/rlk_oracle.c) gives for them.

    python tests/golden/make_vectors.py

Inputs come from numpy's PCG64 with fixed seeds and are rounded to bf16-representable values, so the
same numbers can be fed to the 16-bit GPU path without a second rounding.  The file guards the oracle
against drift (CPU test) and gives the HIP path a committed target (GPU test).
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import c_oracle  # noqa: E402


def bf16_round(x):
    """Round-to-nearest-even to the bf16 grid, returned as float32."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


CASES = {
    # name: (seed, tokens, hidden, vocab, temperature, bias?, ignore every k-th token or 0)
    "small_tail": (11, 37, 64, 300, 1.0, False, 0),
    "temp_bias_ignore": (12, 70, 64, 515, 0.7, True, 9),
    "two_tiles": (13, 300, 32, 520, 1.3, False, 50),
}


def main():
    c_oracle.build(force=False)
    out = {}
    for name, (seed, n, h, v, temp, use_bias, ign_k) in CASES.items():
        rng = np.random.Generator(np.random.PCG64(seed))
        hidden = bf16_round(rng.standard_normal((n, h)))
        weight = bf16_round(rng.standard_normal((v, h)) * 0.05)
        bias = (rng.standard_normal(v) * 0.1).astype(np.float32) if use_bias else None
        targets = rng.integers(0, v, n).astype(np.int64)
        if ign_k:
            targets[::ign_k] = -100
        grad = rng.standard_normal(n).astype(np.float32)
        ign = -100 if ign_k else None
        logp, lse = c_oracle.linear_logp(hidden, weight, targets, bias, temperature=temp,
                                         ignore_index=ign)
        dh, dw, db = c_oracle.linear_logp_backward(grad, hidden, weight, targets, bias,
                                                   temperature=temp, ignore_index=ign)
        out.update({f"{name}/hidden": hidden, f"{name}/weight": weight, f"{name}/targets": targets,
                    f"{name}/grad": grad, f"{name}/temperature": np.float64(temp),
                    f"{name}/logp": logp, f"{name}/lse": lse, f"{name}/dh": dh.astype(np.float32),
                    f"{name}/dw": dw.astype(np.float32)})
        if use_bias:
            out[f"{name}/bias"] = bias
            out[f"{name}/db"] = db
    # GRPO epilogue: 6 sequences x 17 positions, two groups of 3
    rng = np.random.Generator(np.random.PCG64(21))
    b, t = 6, 17
    cur = -np.abs(rng.standard_normal((b, t))).astype(np.float32)
    old = (cur + 0.3 * rng.standard_normal((b, t))).astype(np.float32)
    ref = (cur + 0.3 * rng.standard_normal((b, t))).astype(np.float32)
    rewards = rng.standard_normal(b).astype(np.float32)
    lens = rng.integers(5, t + 1, b)
    mask = (np.arange(t)[None, :] < lens[:, None])
    adv = c_oracle.group_advantages(rewards, [0, 3, 6])
    adv_tok = np.repeat(adv[:, None], t, axis=1)
    out3, dcur = c_oracle.grpo_from_logp(cur, old, ref, adv_tok, mask, clip_eps=0.2, beta=0.04)
    out.update({"grpo/cur": cur, "grpo/old": old, "grpo/ref": ref, "grpo/rewards": rewards,
                "grpo/mask": mask, "grpo/adv": adv, "grpo/out3": out3,
                "grpo/dcur": np.asarray(dcur).reshape(b, t)})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "seeded_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
