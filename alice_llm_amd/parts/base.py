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

    keep_stored: on the bfloat16 path a matrix that its file stores in 32-bit is rounded to bfloat16 once, at
    load, so that it runs on the matrix cores like any other (the reference converts its stored formats once at
    load too, llama3.rs:12889-12890, 18226-18240); with keep_stored it stays 32-bit and its products run on the
    plain kernel.  Norm weights always stay as stored.
    """
    name: str
    act: torch.dtype
    full: bool
    keep_stored: bool = False

    @staticmethod
    def of(name, keep_stored: bool = False) -> "Precision":
        if isinstance(name, Precision):
            return name
        key = {"bf16": "bfloat16", "fp32": "float32", torch.bfloat16: "bfloat16",
               torch.float32: "float32"}.get(name, name)
        if key == "bfloat16":
            return Precision("bfloat16", torch.bfloat16, False, bool(keep_stored))
        if key == "float32":
            return Precision("float32", torch.float32, True, bool(keep_stored))
        raise ValueError(f"unknown dtype '{name}': bfloat16 or float32")

    def matrix(self, w: torch.Tensor) -> torch.Tensor:
        """A matrix weight in the dtype in which this run keeps it: as stored, except that the bfloat16 path
        rounds a matrix stored in 32-bit to bfloat16 (unless keep_stored)."""
        if self.name == "bfloat16" and not self.keep_stored and w.dtype == torch.float32:
            return w.to(torch.bfloat16)
        return w


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
    """Keys and values that grow with the sequence: per position, num_kv_heads rows of head_dim keys and of
    value_head_dim values (None: the same as the keys); `window` keys back from the newest are ever read
    (None: all of them).  `page_size`: the number of positions per page that the mixer's kernels are written
    for (None: any); a cache built with another page size refuses the mixer when the model is put together.
    `dtype`: the dtype of the pages (None: the run's activation dtype); a mixer that wants its keys in 32-bit
    under bfloat16 activations says so here, and its layers get storage of their own."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_head_dim: Optional[int] = None
    page_size: Optional[int] = None
    dtype: Optional[torch.dtype] = None

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_head_dim is None else self.value_head_dim


@dataclass(frozen=True)
class StateNeed:
    """One tensor of fixed size per sequence, zero when the sequence starts.  A mixer may declare several
    (a convolution tail and a recurrent matrix, say); it finds each under its name in LayerCache.state."""
    name: str
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass(frozen=True)
class CacheNeed:
    kv: Optional[KVNeed] = None
    state: Tuple[StateNeed, ...] = ()

    def __post_init__(self):
        st = self.state
        if isinstance(st, StateNeed):
            st = (st,)
        st = tuple(st or ())
        names = [s.name for s in st]
        if len(set(names)) != len(names):
            raise ValueError(f"state tensors of one part need distinct names, found {names}")
        object.__setattr__(self, "state", st)


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
