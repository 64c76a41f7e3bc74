"""A causal language model put together from a plan: embedding, layers of parts run in the order
of the schedule, final norm, output head.  This file knows no architecture; the reference's
counterpart is one forward with per-architecture switches (llama3.rs:13632-14614).
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, List, Optional, Tuple

import torch

from ..config.plan import ModelPlan, PartSpec
from ..parts import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, ParamSpec, Precision,
                     ResidualStream)


class Layer:
    def __init__(self, plan_layer, precision: Precision, positions: dict):
        self.prefix = plan_layer.prefix
        self.mixer = MIXERS.get(plan_layer.mixer.kind)(precision, positions, **plan_layer.mixer.args)
        self.feed_forward = FEED_FORWARDS.get(plan_layer.feed_forward.kind)(precision, **plan_layer.feed_forward.args)
        self.norms = {role: NORMS.get(spec.kind)(precision, **spec.args) for role, spec in plan_layer.norms.items()}
        self.block = BLOCKS.get(plan_layer.block)(self.mixer, self.feed_forward, self.norms)
        self._named = [(plan_layer.mixer.name, self.mixer), (plan_layer.feed_forward.name, self.feed_forward)]
        self._named += [(plan_layer.norms[role].name, n) for role, n in self.norms.items()]

    def named_parts(self):
        return [(self.prefix + name + ".", part) for name, part in self._named]


class CausalLM:
    def __init__(self, plan: ModelPlan, precision, device):
        self.plan = plan
        self.precision = Precision.of(precision)
        self.device = torch.device(device)
        p = self.precision
        self.positions = {name: POSITIONS.get(spec.kind)(p, self.device, **spec.args)
                          for name, spec in plan.positions.items()}
        if "none" not in self.positions:
            self.positions["none"] = POSITIONS.get("none")(p, self.device)
        self.embedding = EMBEDDINGS.get(plan.embedding.kind)(p, **plan.embedding.args)
        self.layers: List[Layer] = [Layer(lp, p, self.positions) for lp in plan.layers]
        self.final_norm = NORMS.get(plan.final_norm.kind)(p, **plan.final_norm.args) if plan.final_norm else None
        self.head = HEADS.get(plan.head.kind)(p, **plan.head.args)
        for e in plan.schedule:
            if not 0 <= e.layer < len(self.layers) or (e.cache_from is not None
                                                       and not 0 <= e.cache_from < len(self.layers)):
                raise ValueError(f"schedule entry {e} names a layer that does not exist")
        self._loaded = False

    # ------------------------------------------------------------------ parameters
    def named_parts(self) -> List[Tuple[str, object]]:
        out = [(self.plan.embedding.name + ".", self.embedding)]
        for layer in self.layers:
            out += layer.named_parts()
        if self.final_norm is not None:
            out.append((self.plan.final_norm.name + ".", self.final_norm))
        out.append((self.plan.head.name + ".", self.head))
        return out

    def param_specs(self) -> "OrderedDict[str, ParamSpec]":
        """Every tensor the model wants, by full name, in a fixed order (the order of random initialisation)."""
        specs: "OrderedDict[str, ParamSpec]" = OrderedDict()
        for prefix, part in self.named_parts():
            for local, spec in part.param_specs().items():
                specs[prefix + local] = spec
        return specs

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        for prefix, part in self.named_parts():
            if name.startswith(prefix) and name[len(prefix):] in part.param_specs():
                part.assign(name[len(prefix):], tensor)
                return
        raise KeyError(name)

    def finalize(self) -> None:
        for _, part in self.named_parts():
            part.finalize()
        tied = getattr(self.head, "tied_to", None)
        if tied:
            if tied != self.plan.embedding.name:
                raise ValueError(f"the head is tied to '{tied}', which is not the embedding")
            self.head.tie(self.embedding)
        self._loaded = True

    def weight_bytes(self) -> int:
        """Bytes of weights a step reads once (tied matrices counted once)."""
        total = 0
        for _, part in self.named_parts():
            if hasattr(part, "weight_bytes"):
                total += part.weight_bytes()
            elif getattr(part, "weight", None) is not None:
                total += part.weight.numel() * part.weight.element_size()
        return total

    # ------------------------------------------------------------------ cache needs
    def cache_needs(self):
        return [layer.mixer.cache_need() if hasattr(layer.mixer, "cache_need") else None for layer in self.layers]

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, cache, block_tables) -> torch.Tensor:
        """Runs the step's tokens through the schedule; returns float32 logits at ctx.want_rows."""
        if not self._loaded:
            raise RuntimeError("the model has no weights yet")
        stream = ResidualStream(self.embedding.forward(ctx.tokens), self.precision)
        for entry in self.plan.schedule:
            view = cache.view(entry.layer, block_tables, read_from=entry.cache_from)
            self.layers[entry.layer].block.forward(stream, ctx, view)
        if ctx.want_rows is None or ctx.want_rows.numel() == 0:
            stream.flush()
            return torch.empty((0, self.plan.vocab_size), dtype=torch.float32, device=self.device)
        normed = stream.rows_normed(self.final_norm, ctx.want_rows)
        return self.head.forward(normed)
