"""Token choice: greedy and temperature sampling.

The reference samples greedily only, with the lowest index on ties
(/root/reference/src/kernels/argmax.cu:12-20). Temperature sampling draws from
softmax(logits / temperature) by inverse CDF; its uniform number comes from a counter
hash of (seed, index of the token among the request's outputs), so what a request
samples does not depend on how it was batched or cut into steps.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..kernels import ops

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform01(seed: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits (exact in fp32) for output ``index`` of a
    request sampled with ``seed``."""
    h = _splitmix64(_splitmix64(seed & _MASK) ^ (index & _MASK))
    return (h >> 40) / float(1 << 24)


@dataclass
class SamplingParams:
    temperature: float = 0.0            # 0: greedy
    seed: int = 0
    max_new_tokens: int = 8             # the reference's default (/root/reference/include/constants.h:14)
    ignore_eos: bool = False

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be >= 1")


class Sampler:
    """Chooses one token for each row of logits on the device."""

    def __init__(self, device, max_rows: int = 64):
        self.device = torch.device(device)
        self._cap = 0
        self._turn = 0
        self._grow(max_rows)

    def _grow(self, n: int) -> None:
        if n <= self._cap:
            return
        self._cap = max(n, 2 * self._cap)
        on_gpu = self.device.type == "cuda"
        # two pinned buffers in turn: the host fills one while the copy out of the other may still be queued
        self._h = [torch.empty((2, self._cap), dtype=torch.float32, pin_memory=on_gpu) for _ in range(2)]
        self._copied = [torch.cuda.Event() if on_gpu else None for _ in range(2)]
        self._d = torch.empty((2, self._cap), dtype=torch.float32, device=self.device)
        self._out = torch.empty(self._cap, dtype=torch.int32, device=self.device)

    def choose(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: Sequence[float],
               out: torch.Tensor) -> None:
        """Queues the choice of one token per row of ``logits`` into ``out`` (int32, on the device)
        and returns without waiting for it."""
        n = logits.shape[0]
        assert len(temperatures) == n and len(uniforms) == n and out.numel() >= n
        if all(t <= 0 for t in temperatures):
            ops.argmax(logits, out[:n])
            return
        self._grow(n)
        self._turn ^= 1
        h, copied = self._h[self._turn], self._copied[self._turn]
        if copied is not None:
            copied.synchronize()          # the copy that last read this buffer is done
        hv = h.numpy()
        hv[0, :n] = temperatures
        hv[1, :n] = uniforms
        self._d.copy_(h, non_blocking=True)
        if copied is not None:
            copied.record()
        ops.sample(logits, self._d[0], self._d[1], out[:n])

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: Sequence[float]) -> List[int]:
        n = logits.shape[0]
        self._grow(n)
        self.choose(logits, temperatures, uniforms, self._out)
        return self._out[:n].tolist()
