"""The architecture-neutral description of a model that the builder consumes.

An architecture's typed configuration turns itself into a ModelPlan: which
parts each layer is made of, with which constants, under which tensor names,
and in which order the layers run.  Nothing below this file knows an
architecture's name.  The reference reaches the same end with `match arch`
switches inside one forward (llama3.rs:13639-13676) and per-layer helper
queries on its configuration (llama3.rs:4634-4726); here the per-layer answers
are data.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A configuration key is missing, of the wrong type, or out of range."""


@dataclass(frozen=True)
class PartSpec:
    """One part: its registry name, its constants, and its tensor-name component."""
    kind: str
    args: Mapping[str, Any] = field(default_factory=dict)
    name: str = ""


@dataclass(frozen=True)
class LayerPlan:
    """One layer: an arrangement (block) of a mixer, a feed-forward and norms.

    `norms` is keyed by the role the block gives each norm, e.g. "pre_mixer",
    "post_mixer", "pre_ff", "post_ff"; a block uses the roles it knows and
    treats an absent one as no norm at that place.
    """
    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Mapping[str, PartSpec]
    prefix: str


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  Every run owns cache storage of its own (a layer named twice keeps two
    caches, one per run), unless `cache_from` names an earlier entry of the schedule, by its index,
    whose cache this run reads instead of writing one (the reference's kv_layer_map,
    llama3.rs:4739-4745)."""
    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelPlan:
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    positions: Mapping[str, PartSpec]
    layers: Tuple[LayerPlan, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    stop_token_ids: Tuple[int, ...] = ()


# --------------------------------------------------------------------------- typed reads

_MISSING = object()


def read_key(d: Mapping[str, Any], key: str, typ, default=_MISSING, *, allow_none=False):
    """Read `key` from a parsed config.json with a type check.

    Unknown keys are ignored by the callers, missing optional keys take their
    default, and a present key of the wrong type is an error: the policy of the
    reference's only config.json reader (llama3.rs:536-589).
    """
    if key not in d:
        if default is _MISSING:
            raise ConfigError(f"config.json: required key '{key}' is missing")
        return default
    v = d[key]
    if v is None:
        if allow_none:
            return None
        if default is not _MISSING:
            return default
        raise ConfigError(f"config.json: key '{key}' is null")
    if typ is float and isinstance(v, int) and not isinstance(v, bool):
        v = float(v)
    if typ is int and isinstance(v, bool):
        raise ConfigError(f"config.json: key '{key}' must be an integer, found {v!r}")
    if not isinstance(v, typ):
        raise ConfigError(f"config.json: key '{key}' must be {typ.__name__}, found {v!r}")
    return v


def require(cond: bool, message: str) -> None:
    if not cond:
        raise ConfigError("config.json: " + message)
