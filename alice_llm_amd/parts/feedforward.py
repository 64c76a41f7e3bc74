"""Feed-forwards.  Gated MLP: down( act(gate x) * (up x) ), the activation on the gate branch
(llama3.rs:14519-14540); for Gemma 2 the activation is the tanh form of GELU
(llama3.rs:6183-6186).  gate and up are stacked into one matrix at load so that one kernel reads
the input once and applies the activation and the product in its epilogue.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..hip import ops
from .base import FEED_FORWARDS, ParamSpec, Part, Precision
from .linear import Linear

_GATED_EPILOGUES = {"gelu_tanh": ops.EPI_GEGLU}


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, hidden_size: int, intermediate_size: int, activation: str):
        if activation not in _GATED_EPILOGUES:
            raise ValueError(f"gated_mlp has no kernel for activation '{activation}'; "
                             f"available: {sorted(_GATED_EPILOGUES)}")
        self.precision = precision
        self.H, self.I = hidden_size, intermediate_size
        self.gate_up = Linear(hidden_size, intermediate_size, precision, epilogue=_GATED_EPILOGUES[activation])
        self.down = Linear(intermediate_size, hidden_size, precision)
        self._parts: Dict[str, torch.Tensor] = {}

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"gate_proj.weight": ParamSpec((self.I, self.H)),
                "up_proj.weight": ParamSpec((self.I, self.H)),
                "down_proj.weight": ParamSpec((self.H, self.I))}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name == "down_proj.weight":
            self.down.load(tensor)
        elif name in ("gate_proj.weight", "up_proj.weight"):
            self._parts[name] = tensor
        else:
            raise KeyError(name)

    def finalize(self) -> None:
        g, u = (self.precision.matrix(self._parts.pop(n + "_proj.weight")) for n in ("gate", "up"))
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.gate_up.load(torch.cat([g, u], dim=0))

    def weight_bytes(self) -> int:
        return self.gate_up.nbytes() + self.down.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return self.gate_up.accepts_fragment_input

    def forward(self, x, ctx) -> torch.Tensor:
        # decode steps: the gated product goes to the down projection in fragment order as well
        frag = (getattr(ctx, "fragment_activations", False) and self.down.accepts_fragment_input
                and self.gate_up.can_write_fragments(x.shape[0]))
        h = self.gate_up(x, self.precision.act, out_fragments=frag)
        return self.down(h, torch.float32, allow_partials=True)
