"""What every part is: declared parameters, constants as constructor arguments, and registries.

A part never learns which model it is in.  It is chosen layer by layer through its registry name
in the plan, receives its sizes and constants as keyword arguments, declares the tensors it wants
under local names ("q_proj.weight"), and declares what it needs from the cache.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

import torch


# --------------------------------------------------------------------------- precision

@dataclass(frozen=True)
class Precision:
    """The arithmetic of a run.

    bfloat16: matrix operands, activations between kernels and the cache are bfloat16; sums,
    softmax, norms, rotation and the residual stream are 32-bit.
    float32: everything is 32-bit, with full-precision tanh/exp/sqrt and no matrix-core shortcut.
    """
    name: str
    act: torch.dtype
    full: bool

    @staticmethod
    def of(name) -> "Precision":
        if isinstance(name, Precision):
            return name
        key = {"bf16": "bfloat16", "fp32": "float32", torch.bfloat16: "bfloat16",
               torch.float32: "float32"}.get(name, name)
        if key == "bfloat16":
            return Precision("bfloat16", torch.bfloat16, False)
        if key == "float32":
            return Precision("float32", torch.float32, True)
        raise ValueError(f"unknown dtype '{name}': bfloat16 or float32")


# --------------------------------------------------------------------------- activations in fragment order

class FragmentActs:
    """bfloat16 activations [rows, cols] stored in the order in which the matrix-core kernels read them
    ([rows/16][cols/32][64 lanes][8], rows padded to 16): a wave fetches a whole operand tile with one
    contiguous 1 KB read instead of sixteen pieces of 64 bytes.  Only parts that declare
    `accepts_fragment_activations` are ever handed one; everything else sees plain tensors."""

    def __init__(self, data: torch.Tensor, rows: int, cols: int):
        self.data, self.rows, self.cols = data, rows, cols

    @property
    def shape(self):
        return (self.rows, self.cols)

    @property
    def device(self):
        return self.data.device

    @staticmethod
    def possible(precision: "Precision", rows: int, cols: int) -> bool:
        return precision.act == torch.bfloat16 and rows >= 1 and cols % 32 == 0

    @staticmethod
    def empty(rows: int, cols: int, device) -> "FragmentActs":
        padded = -(-rows // 16) * 16
        return FragmentActs(torch.empty(padded * cols, dtype=torch.bfloat16, device=device), rows, cols)


# --------------------------------------------------------------------------- parameters

@dataclass(frozen=True)
class ParamSpec:
    """A tensor a part wants: its shape, the standard deviation of its random initialisation, and
    whether it is a floating-point weight (kept bfloat16 or float32 as stored) or an integer table
    (kept int32)."""
    shape: Tuple[int, ...]
    init_std: float = 0.02
    integer: bool = False


class Part:
    """Base of all parts.  Subclasses list parameters in `param_specs`, take them in `assign`
    (already on the device, in their stored dtype), and may fuse or rearrange them in `finalize`."""

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        raise KeyError(name)

    def finalize(self) -> None:
        pass


# --------------------------------------------------------------------------- cache needs

@dataclass(frozen=True)
class KVNeed:
    """Keys and values that grow with the sequence: rows of num_kv_heads x head_dim per position;
    `window` keys back from the newest are ever read (None: all of them)."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size per sequence, zero when the sequence starts."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass(frozen=True)
class CacheNeed:
    kv: Optional[KVNeed] = None
    state: Optional[StateNeed] = None


# --------------------------------------------------------------------------- registries

class Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: Dict[str, Callable] = {}

    def register(self, name: str, item: Callable = None):
        """Use as `REG.register("name", cls)` or as a decorator `@REG.register("name")`."""
        if item is not None:
            self._items[name] = item
            return item

        def deco(cls):
            self._items[name] = cls
            return cls
        return deco

    def get(self, name: str) -> Callable:
        if name not in self._items:
            raise KeyError(f"unknown {self.what} '{name}'; registered: {sorted(self._items)}")
        return self._items[name]

    def names(self) -> List[str]:
        return sorted(self._items)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITIONS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")
