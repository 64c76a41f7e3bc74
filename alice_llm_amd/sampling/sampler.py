"""Greedy and temperature sampling, top-k and top-p, with a counter-based random stream per request.

Semantics follow the reference's sampling functions (src/sampling.rs:10-123) in the order its
drivers apply them, temperature -> top-k -> softmax -> draw, greedy below a temperature of 1e-6
(examples/generate_gpu.rs:122-129).  The uniform number of request r at its n-th draw is a
function of (seed, r, n) alone (SplitMix64 as in llama3.rs:19109-19129, top 24 bits), so a
request's tokens do not depend on which other requests share its batch.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..hip import ops

_M = (1 << 64) - 1
GREEDY_BELOW = 1e-6


def splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _M
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M
    return z ^ (z >> 31)


def uniform(seed: int, request: int, n: int) -> float:
    """The n-th uniform number in [0, 1) of request `request` under `seed`."""
    stream = splitmix64((seed & _M) ^ ((request * 0xD1B54A32D192ED03) & _M))
    return (splitmix64((stream + n) & _M) >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, seed: int = 0):
        if temperature < 0:
            raise ValueError("temperature must not be negative")
        if top_k < 0:
            raise ValueError("top_k must not be negative (0 turns it off)")
        if not top_p > 0:
            raise ValueError("top_p must be positive (1 turns it off)")
        self.temperature, self.top_k, self.top_p, self.seed = float(temperature), int(top_k), float(top_p), int(seed)

    @property
    def greedy(self) -> bool:
        return self.temperature < GREEDY_BELOW

    def __call__(self, logits: torch.Tensor, requests: Sequence[int], draws: Sequence[int]) -> torch.Tensor:
        """logits: float32 [B, V] on the GPU; requests[i], draws[i]: which request row i belongs to and
        how many tokens it has drawn before.  Returns int32 [B] on the GPU."""
        if self.greedy:
            return ops.argmax(logits)
        u = torch.tensor([uniform(self.seed, r, n) for r, n in zip(requests, draws)], dtype=torch.float32)
        return ops.sample(logits, u.to(logits.device), self.temperature, self.top_k, self.top_p)
