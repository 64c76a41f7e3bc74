"""Position encodings.  Rotary, half-split pairing (j, j + R/2) over the rotated width R:
angle = position * theta^(-2j/R) (llama3.rs:5367-5378; same pairing in src/rope.rs:12-27).

The angles' cosines and sines are tabulated once on the host in 64-bit and stored as 32-bit, so
the rotation itself is a 32-bit multiply-add in the kernel.  A position encoding serves the
attention mixer through `rotate_and_store`: rotate q and k, and put k and v into the cache in the
same pass, which saves one trip through memory for k.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..hip import ops
from .base import POSITIONS, Part, Precision


@POSITIONS.register("rope")
class RotaryEncoding(Part):
    graph_safe = True

    def __init__(self, precision: Precision, device, *, dim: int, theta: float, max_positions: int,
                 rotary_dim: Optional[int] = None):
        self.dim = dim
        self.rotary_dim = dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or self.rotary_dim > dim:
            raise ValueError(f"rotated width {self.rotary_dim} must be even and at most {dim}")
        self.theta = float(theta)
        self.max_positions = max_positions
        half = self.rotary_dim // 2
        j = torch.arange(half, dtype=torch.float64)
        inv_freq = self.theta ** (-2.0 * j / self.rotary_dim)
        ang = torch.arange(max_positions, dtype=torch.float64)[:, None] * inv_freq[None, :]
        self.cos = torch.cos(ang).to(torch.float32).to(device).contiguous()
        self.sin = torch.sin(ang).to(torch.float32).to(device).contiguous()

    def projection_row_order(self, num_heads: int, num_kv_heads: int, head_dim: int) -> Optional[torch.Tensor]:
        """A mixer that fuses its q, k and v projections may put the rows of every q and k head in pair order
        (rows j and j + d/2 at 2j and 2j + 1): the two elements of a rotated pair then leave the matrix product
        next to each other, in one lane of one tile, and the rotation can be its epilogue.  Returns the row
        permutation of the fused [q | k | v] matrix, or None where this does not apply (a partly rotated head).
        The mixer then passes pair_order=True to rotate_and_store."""
        if self.rotary_dim != head_dim or head_dim != self.dim or head_dim % 2:
            return None
        half = head_dim // 2
        one = torch.stack([torch.arange(half), torch.arange(half) + half], dim=1).flatten()      # 0, half, 1, half+1, ..
        heads = torch.arange(num_heads + num_kv_heads)[:, None] * head_dim + one[None, :]
        v0 = (num_heads + num_kv_heads) * head_dim
        return torch.cat([heads.flatten(), torch.arange(v0, v0 + num_kv_heads * head_dim)])

    def rotate_and_store(self, qkv: torch.Tensor, q_out: torch.Tensor, ctx, cache, *, num_heads: int,
                         num_kv_heads: int, head_dim: int, kv_layout: int = 0, pair_order: bool = False) -> None:
        write = cache is not None and cache.writable
        ops.rope_cache_write(qkv, q_out, cache.k if write else None, cache.v if write else None,
                             self.cos, self.sin, ctx.positions, ctx.seq_of_token if write else None,
                             cache.block_table if write else None, num_heads=num_heads,
                             num_kv_heads=num_kv_heads, head_dim=head_dim, rotary_dim=self.rotary_dim,
                             max_position=ctx.max_position, kv_layout=kv_layout, interleaved=pair_order)

    def project_rotate_store(self, proj, x, q_out: torch.Tensor, ctx, cache, *, num_heads: int, num_kv_heads: int,
                             head_dim: int, kv_layout: int) -> bool:
        """Projection (a Linear in the fragment layout with its rows in pair order), rotation and cache write as
        one kernel.  False where that kernel does not apply; the caller then takes the steps apart."""
        from .base import FragmentActs
        frag_in = isinstance(x, FragmentActs)
        if not (cache is not None and cache.writable
                and proj.layout == ops.LAYOUT_FRAG16 and proj.precision.act == torch.bfloat16 and head_dim % 16 == 0
                and (kv_layout == ops.KV_ROW or head_dim % 32 == 0)):
            return False
        ops.linear_rope_cache(x.data if frag_in else x, proj.weight, q_out, cache.k, cache.v, self.cos, self.sin,
                              ctx.positions, ctx.seq_of_token, cache.block_table, k_in=proj.k, num_heads=num_heads,
                              num_kv_heads=num_kv_heads, head_dim=head_dim, max_position=ctx.max_position,
                              kv_layout=kv_layout, rows=x.shape[0],
                              x_layout=ops.LAYOUT_FRAG16 if frag_in else ops.LAYOUT_ROW)
        return True


@POSITIONS.register("none")
class NoPositionEncoding(Part):
    graph_safe = True

    """No rotation: q passes through, k and v go to the cache unchanged."""

    def __init__(self, precision: Precision, device, **_):
        pass

    def rotate_and_store(self, qkv, q_out, ctx, cache, *, num_heads, num_kv_heads, head_dim, kv_layout=0) -> None:
        write = cache is not None and cache.writable
        ops.rope_cache_write(qkv, q_out, cache.k if write else None, cache.v if write else None, None, None,
                             ctx.positions, ctx.seq_of_token if write else None,
                             cache.block_table if write else None, num_heads=num_heads,
                             num_kv_heads=num_kv_heads, head_dim=head_dim, rotary_dim=0,
                             max_position=ctx.max_position, kv_layout=kv_layout)
