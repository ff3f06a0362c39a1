"""Choosing the next token from logits.

Greedy is the reference's rule: the first index of the maximum
(src/engine.cpp:52-58). The reference samples in no other way; temperature
sampling here is p = softmax(logits / T), token = first id whose cumulative
probability (ascending ids) exceeds u * sum(p). The draw u comes from a
counter-based generator keyed by (seed, request, index of the generated token), so
what a request samples does not depend on what else is in its batch.
"""
from __future__ import annotations

from typing import Sequence

import torch

from .. import ops

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform_draw(seed: int, request: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits (exact in 32-bit floats)."""
    x = _splitmix64(int(seed) & _MASK)
    x = _splitmix64(x ^ (int(request) & _MASK))
    x = _splitmix64(x ^ (int(index) & _MASK))
    return (x >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, temperature: float = 0.0, seed: int = 0):
        if temperature < 0:
            raise ValueError("temperature must be >= 0")
        self.temperature = float(temperature)
        self.seed = int(seed)
        self._device_rows: dict = {}            # (device, rows) -> ([2, rows] temperatures and draws, pinned draws)

    def choose(self, logits: torch.Tensor, draws: Sequence[tuple[int, int]] | None = None) -> list[int]:
        """One token per row of logits [R, V] (32-bit, on the device). `draws` gives
        (request, index) per row for the random draw; not needed when greedy."""
        R = logits.shape[0]
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
        if self.temperature == 0.0:
            ops.argmax(logits, out)
        else:
            if draws is None or len(draws) != R:
                raise ValueError("temperature sampling needs a (request, index) pair per row")
            # the temperatures stay on the device from one step to the next; only the draws go up
            # (from pinned memory, so the copy does not wait; the tokens' read-back below ends
            # the step before the next one writes the pinned row again)
            key = (logits.device, R)
            held = self._device_rows.get(key)
            if held is None:
                rows = torch.empty(2, R, dtype=torch.float32, device=logits.device)
                rows[0].fill_(self.temperature)
                held = self._device_rows[key] = (rows, torch.empty(R, dtype=torch.float32, pin_memory=True))
            rows, pinned = held
            pinned.copy_(torch.tensor([uniform_draw(self.seed, r, i) for r, i in draws], dtype=torch.float32))
            rows[1].copy_(pinned, non_blocking=True)
            ops.sample(logits, rows[0], rows[1], out)
        return out.tolist()
