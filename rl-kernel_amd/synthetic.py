"""Counter-based synthetic inputs for the benchmark and the full-size tests: the value of element
``i`` of tensor ``tensor_id`` under ``seed`` is a pure function of ``(seed, tensor_id, i)``, computed
in integer arithmetic, so a CPU run and a GPU run (any torch / rocRAND build) produce the same bits.

    key    = splitmix64(splitmix64(seed) + tensor_id)
    h_k(i) = splitmix64(key + 3 i + k),  k = 0, 1, 2          (three 64-bit hashes per element)
    normal = (sum of the twelve 16-bit lanes of h_0..h_2 - 6 * 65535) / 65536
             (Irwin-Hall: mean 0, variance 1 to 2^-32, support +-6; every value is exact in fp32)
    index  = (h_0(i) >> 1) mod n

The role of the reference's ``make_synthetic_rl_kernel_batch``
(rl_engine/testing/rl_batch.py:118-168), whose values depend on the draw order of a torch
Generator; the distributions here are the ones the benchmark configurations state.
"""

from __future__ import annotations

from typing import Sequence

import torch

_GOLDEN = -7046029254386353131      # 0x9E3779B97F4A7C15 as a signed 64-bit integer
_M1 = -4658895280553007687          # 0xBF58476D1CE4E5B9
_M2 = -7723592293110705685          # 0x94D049BB133111EB


def _lsr(x: torch.Tensor, n: int) -> torch.Tensor:
    """Logical shift right of int64 lanes (torch's >> is arithmetic)."""
    return (x >> n) & ((1 << (64 - n)) - 1)


def splitmix64(x: torch.Tensor) -> torch.Tensor:
    """One splitmix64 step on int64 lanes (two's-complement wrap-around arithmetic)."""
    z = x + _GOLDEN
    z = (z ^ _lsr(z, 30)) * _M1
    z = (z ^ _lsr(z, 27)) * _M2
    return z ^ _lsr(z, 31)


def _key(seed: int, tensor_id: int, device) -> torch.Tensor:
    s = torch.tensor([seed], dtype=torch.int64, device=device)
    return splitmix64(splitmix64(s) + tensor_id)


def _hashes(seed: int, tensor_id: int, start: int, count: int, device, k: int) -> torch.Tensor:
    idx = torch.arange(start, start + count, dtype=torch.int64, device=device)
    return splitmix64(_key(seed, tensor_id, device) + 3 * idx + k)


def normal(seed: int, tensor_id: int, shape: Sequence[int], *, std: float = 1.0,
           dtype: torch.dtype = torch.float32, device="cpu", chunk: int = 1 << 24) -> torch.Tensor:
    """``shape`` values ~ N(0, std^2) (Irwin-Hall of 12), rounded once to ``dtype``."""
    numel = 1
    for s in shape:
        numel *= int(s)
    out = torch.empty(numel, dtype=dtype, device=device)
    for start in range(0, numel, chunk):
        count = min(chunk, numel - start)
        total = torch.zeros(count, dtype=torch.int64, device=device)
        for k in range(3):
            h = _hashes(seed, tensor_id, start, count, device, k)
            for lane in range(4):
                total += _lsr(h, 16 * lane) & 0xFFFF
        z = (total - 6 * 65535).to(torch.float32) / 65536.0      # exact in fp32
        out[start:start + count] = (z * std).to(dtype) if std != 1.0 else z.to(dtype)
    return out.reshape(*shape)


def randint(seed: int, tensor_id: int, shape: Sequence[int], high: int, *, device="cpu") -> torch.Tensor:
    """``shape`` int64 values in ``[0, high)``."""
    numel = 1
    for s in shape:
        numel *= int(s)
    h = _hashes(seed, tensor_id, 0, numel, device, 0)
    return (_lsr(h, 1) % int(high)).reshape(*shape)


def bernoulli(seed: int, tensor_id: int, shape: Sequence[int], p: float, *, device="cpu") -> torch.Tensor:
    """``shape`` booleans, true with probability ``p`` (24-bit resolution)."""
    numel = 1
    for s in shape:
        numel *= int(s)
    h = _hashes(seed, tensor_id, 0, numel, device, 0)
    return ((_lsr(h, 40)) < int(p * (1 << 24))).reshape(*shape)
