"""Token embedding and the output head.

Embedding: x = E[token] * scale, a row copy into the 32-bit residual stream (llama3.rs:13686-13703;
for Gemma 2 the plan passes scale = sqrt(width) rounded to f32).  Head: logits = softcap(W n) in
float32 (llama3.rs:14602-14611), W being the embedding matrix itself when the head is tied
(llama3.rs:12896-12906): one matrix on the device serves both.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..hip import ops
from .base import EMBEDDINGS, HEADS, ParamSpec, Part, Precision
from .linear import Linear


@EMBEDDINGS.register("embedding")
class Embedding(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, vocab_size: int, dim: int, scale: float = 1.0):
        self.precision = precision
        self.V, self.dim, self.scale = vocab_size, dim, float(scale)
        self.table = Linear(dim, vocab_size, precision)     # stored as the head reads it

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.V, self.dim))}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name != "weight":
            raise KeyError(name)
        self.table.load(tensor)

    def weight_bytes(self) -> int:
        return self.table.nbytes()

    def forward(self, ctx) -> torch.Tensor:
        """The float32 rows that start the residual stream, one per token of the step.  An embedding sees the
        whole step (`ctx`: token ids, positions, the sequence of each token), so that one that adds a learned
        row per position, say, needs nothing else; this one reads the ids only."""
        tokens = ctx.tokens
        out = torch.empty((tokens.numel(), self.dim), dtype=torch.float32, device=tokens.device)
        ops.embed(tokens, self.table.weight, out, self.scale, self.V, self.dim, self.table.layout)
        return out


@HEADS.register("lm_head")
class OutputHead(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, vocab_size: int, dim: int, softcap: Optional[float] = None,
                 tied_to: Optional[str] = None):
        self.precision = precision
        self.V, self.dim = vocab_size, dim
        self.softcap = None if softcap is None else float(softcap)
        self.tied_to = tied_to
        self.proj = Linear(dim, vocab_size, precision,
                           epilogue=ops.EPI_SOFTCAP if self.softcap else ops.EPI_NONE,
                           epi_param=self.softcap or 0.0)

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {} if self.tied_to else {"weight": ParamSpec((self.V, self.dim))}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name != "weight" or self.tied_to:
            raise KeyError(name)
        self.proj.load(tensor)

    def tie(self, embedding: Embedding) -> None:
        self.proj.weight = embedding.table.weight
        self.proj.layout = embedding.table.layout

    def weight_bytes(self) -> int:
        return 0 if self.tied_to else self.proj.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return self.proj.accepts_fragment_input

    def forward(self, x) -> torch.Tensor:
        """x: [n, dim] normed rows (a tensor or FragmentActs); returns float32 logits [n, V]."""
        return self.proj(x, torch.float32)
