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
        for i, e in enumerate(plan.schedule):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"schedule entry {i} names layer {e.layer}, which does not exist")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < i or plan.schedule[e.cache_from].cache_from is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_from}, which must be "
                                     f"an earlier entry with a cache of its own")
                a, b = self._need(e.layer), self._need(plan.schedule[e.cache_from].layer)
                if a is None or b is None or a.kv is None or b.kv is None or \
                        (a.kv.num_kv_heads, a.kv.head_dim, a.kv.v_dim, a.kv.dtype) != (b.kv.num_kv_heads, b.kv.head_dim, b.kv.v_dim, b.kv.dtype) or \
                        (b.kv.window is not None and (a.kv.window is None or a.kv.window > b.kv.window)):
                    raise ValueError(f"schedule entry {i} cannot read the cache of entry {e.cache_from}: "
                                     f"its keys differ in shape or dtype, or reach further back than that cache keeps")
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

    def graph_safe(self) -> bool:
        """Whether a decode step of this model can be recorded into a HIP graph: every part that runs in a
        step declares `graph_safe = True` (its launches depend on device data and on sizes fixed per graph)."""
        parts = [self.embedding, self.head, self.final_norm] + list(self.positions.values())
        for layer in self.layers:
            parts += [layer.mixer, layer.feed_forward, layer.block] + list(layer.norms.values())
        return all(getattr(p, "graph_safe", False) for p in parts if p is not None)

    def prompt_graph_safe(self) -> bool:
        """Whether steps of several tokens a sequence can be recorded too: every part that keeps state of its own
        (a cache need with state tensors) declares `graph_safe_prompts = True`, that is, it advances its state
        token by token on the device, from ctx.cu_seqlens and ctx.seq_of_token, never from the host copies."""
        for e in self.plan.schedule:
            need = self._need(e.layer)
            if need is not None and need.state and not getattr(self.layers[e.layer].mixer, "graph_safe_prompts", False):
                return False
        return True

    # ------------------------------------------------------------------ cache needs
    def _need(self, layer: int):
        mixer = self.layers[layer].mixer
        return mixer.cache_need() if hasattr(mixer, "cache_need") else None

    def cache_needs(self):
        """What each entry of the schedule needs from the cache (None for a run that reads another's)."""
        return [None if e.cache_from is not None else self._need(e.layer) for e in self.plan.schedule]

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, cache, block_tables) -> torch.Tensor:
        """Runs the step's tokens through the schedule; returns float32 logits at ctx.want_rows."""
        if not self._loaded:
            raise RuntimeError("the model has no weights yet")
        stream = ResidualStream(self.embedding.forward(ctx), self.precision)
        for i, entry in enumerate(self.plan.schedule):
            view = cache.view(i, block_tables, read_from=entry.cache_from)
            self.layers[entry.layer].block.forward(stream, ctx, view)
        if ctx.want_rows is None or ctx.want_rows.numel() == 0:
            stream.flush()
            return torch.empty((0, self.plan.vocab_size), dtype=torch.float32, device=self.device)
        frag = getattr(ctx, "fragment_activations", False) and getattr(self.head, "accepts_fragment_activations", False)
        if getattr(ctx, "want_every_row", False):
            normed = stream.normed(self.final_norm, fragments=frag)        # the last add and the norm as one kernel
        else:
            normed = stream.rows_normed(self.final_norm, ctx.want_rows, fragments=frag)
        return self.head.forward(normed)
