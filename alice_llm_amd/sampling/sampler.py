"""Greedy and temperature sampling, top-k and top-p, with a counter-based random stream per request.

Semantics follow the reference's sampling functions (src/sampling.rs:10-123) in the order its
drivers apply them, temperature -> top-k -> softmax -> draw, greedy below a temperature of 1e-6
(examples/generate_gpu.rs:122-129).  The uniform number of request r at its n-th draw is a
function of (seed, r, n) alone (SplitMix64 as in llama3.rs:19109-19129, top 24 bits), so a
request's tokens do not depend on which other requests share its batch.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

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
        # pinned host buffers for the uniform numbers, used in turn: their copies are queued behind the step's
        # kernels without the host waiting for them (a copy from ordinary memory would wait)
        self._pinned: List[Optional[torch.Tensor]] = [None] * 4
        self._copied: List[Optional[torch.cuda.Event]] = [None] * 4
        self._turn = 0

    @property
    def greedy(self) -> bool:
        return self.temperature < GREEDY_BELOW

    def __call__(self, logits: torch.Tensor, requests: Sequence[int], draws: Sequence[int]) -> torch.Tensor:
        """logits: float32 [B, V] on the GPU; requests[i], draws[i]: which request row i belongs to and
        how many tokens it has drawn before.  Returns int32 [B] on the GPU."""
        if self.greedy:
            return ops.argmax(logits)
        u = torch.tensor([uniform(self.seed, r, n) for r, n in zip(requests, draws)], dtype=torch.float32)
        return ops.sample(logits, self._upload(u, logits.device), self.temperature, self.top_k, self.top_p)

    def _upload(self, u: torch.Tensor, device) -> torch.Tensor:
        i = self._turn = (self._turn + 1) % len(self._pinned)
        if self._copied[i] is not None:
            self._copied[i].synchronize()                    # the copy that last read this buffer has run
        if self._pinned[i] is None or self._pinned[i].numel() < u.numel():
            self._pinned[i] = torch.empty(max(64, 2 * u.numel()), dtype=torch.float32).pin_memory()
        host = self._pinned[i][:u.numel()]
        host.copy_(u)
        out = torch.empty(u.numel(), dtype=torch.float32, device=device)
        out.copy_(host, non_blocking=True)
        self._copied[i] = torch.cuda.Event()
        self._copied[i].record()
        return out
