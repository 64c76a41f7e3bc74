"""The attention mixer: grouped-query attention over the paged cache.

q, k, v projections (no biases), position encoding of q and k, k and v cached, then per query
head h with kv head h // (nH // nKV): score = (q . k) * scale, softcap cap * tanh(s / cap),
softmax over the keys max(0, pos + 1 - window) .. pos, weighted sum of v, output projection
(llama3.rs:14206-14217, 14307-14331, 5431-5451, 5622-5688, 14423).  Scale, softcap, window, head
counts and head size are constructor arguments; window None is global attention, softcap None
turns the tanh off.  A position term at the score stage is a constructor argument too:
score_bias_slopes, one slope a query head, adds slope * (key position - query position) to the
capped score (a linear distance bias; the 32-bit attention kernel over a row-major cache takes it,
in both dtypes).
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..hip import ops
from .base import MIXERS, CacheNeed, FragmentActs, KVNeed, ParamSpec, Part, Precision
from .linear import Linear


@MIXERS.register("attention")
class Attention(Part):
    graph_safe = True

    def __init__(self, precision: Precision, positions: dict, *, hidden_size: int, num_heads: int,
                 num_kv_heads: int, head_dim: int, scale: float, softcap: Optional[float] = None,
                 window: Optional[int] = None, position: Optional[str] = None,
                 score_bias_slopes: Optional[Sequence[float]] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_kv_heads {num_kv_heads} must divide num_heads {num_heads}")
        if not 1 <= head_dim <= ops.ATTENTION_MAX_HEAD_DIM:
            # refused when the model is put together, not at its first step
            raise ValueError(f"attention: head_dim {head_dim} is outside 1..{ops.ATTENTION_MAX_HEAD_DIM}, the range "
                             f"of the attention kernels")
        self.precision = precision
        self.H, self.nH, self.nKV, self.d = hidden_size, num_heads, num_kv_heads, head_dim
        self.scale = float(scale)
        self.softcap = None if softcap is None else float(softcap)
        self.window = window
        if score_bias_slopes is not None and len(score_bias_slopes) != num_heads:
            raise ValueError(f"attention: {len(score_bias_slopes)} score bias slopes for {num_heads} heads")
        self.score_bias_slopes = None if score_bias_slopes is None else [float(v) for v in score_bias_slopes]
        self._slopes: Optional[torch.Tensor] = None
        self.position = positions[position] if position is not None else positions.get("none")
        if self.position is None:
            raise ValueError("attention needs a position encoding (use 'none' for no rotation)")
        self.q_dim, self.kv_dim = num_heads * head_dim, num_kv_heads * head_dim
        self.qkv = Linear(hidden_size, self.q_dim + 2 * self.kv_dim, precision)
        self.o = Linear(self.q_dim, hidden_size, precision)
        # How this mixer lays keys and values out inside a page: the matrix-core kernels read a fragment
        # layout; every other case is row-major.  It depends on the arithmetic and the head size alone, so
        # that a run that reads another run's cache finds the layout it expects.
        self.kv_layout = (ops.KV_FRAGMENT if precision.name == "bfloat16" and precision.act == torch.bfloat16
                          and ops.library_ready() and ops.attention_mfma_supported(head_dim)
                          and score_bias_slopes is None else ops.KV_ROW)
        self._parts: Dict[str, torch.Tensor] = {}

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"q_proj.weight": ParamSpec((self.q_dim, self.H)),
                "k_proj.weight": ParamSpec((self.kv_dim, self.H)),
                "v_proj.weight": ParamSpec((self.kv_dim, self.H)),
                "o_proj.weight": ParamSpec((self.H, self.q_dim))}

    def cache_need(self) -> CacheNeed:
        # the fragment layout of the matrix-core kernels is written for pages of 64 positions
        page = ops.KV_FRAGMENT_PAGE if self.kv_layout == ops.KV_FRAGMENT else None
        return CacheNeed(kv=KVNeed(self.nKV, self.d, self.window, page_size=page))

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name == "o_proj.weight":
            self.o.load(tensor)
        elif name in ("q_proj.weight", "k_proj.weight", "v_proj.weight"):
            self._parts[name] = tensor
        else:
            raise KeyError(name)

    def finalize(self) -> None:
        q, k, v = (self.precision.matrix(self._parts.pop(n + "_proj.weight")) for n in "qkv")
        if not (q.dtype == k.dtype == v.dtype):
            q, k, v = q.float(), k.float(), v.float()       # kept as stored, one of them in 32-bit: the fused matrix is 32-bit
        w = torch.cat([q, k, v], dim=0)                     # rows: all q heads, then k heads, then v heads
        # a position encoding may ask for the rows of the q and k heads in another order (rotated pairs next to
        # each other), so that its rotation can be the projection's epilogue
        order = getattr(self.position, "projection_row_order", lambda *a: None)(self.nH, self.nKV, self.d)
        self.pair_order = order is not None
        if self.pair_order:
            w = w[order.to(w.device)]
        self.qkv.load(w)
        if self.score_bias_slopes is not None:
            self._slopes = torch.tensor(self.score_bias_slopes, dtype=torch.float32, device=w.device)

    def weight_bytes(self) -> int:
        return self.qkv.nbytes() + self.o.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return self.qkv.accepts_fragment_input

    def forward(self, x, ctx, cache) -> torch.Tensor:
        """x: [T, H] in the activation dtype (a tensor, or FragmentActs in decode steps); returns the branch
        in float32 ([T, H] or partial sums)."""
        T = x.shape[0]
        q = torch.empty((T, self.q_dim), dtype=self.precision.act, device=x.device)
        geometry = dict(num_heads=self.nH, num_kv_heads=self.nKV, head_dim=self.d, kv_layout=self.kv_layout)
        fused = self.pair_order and self.position.project_rotate_store(self.qkv, x, q, ctx, cache, **geometry)
        if not fused:
            qkv = self.qkv(x, self.precision.act)
            if self.pair_order:
                self.position.rotate_and_store(qkv, q, ctx, cache, pair_order=True, **geometry)
            else:
                self.position.rotate_and_store(qkv, q, ctx, cache, **geometry)
        # Single tokens of at most 16 sequences whose keys are split over blocks: the output projection combines the
        # splits itself (one kernel fewer a layer).
        if (ctx.is_decode and self.kv_layout == ops.KV_FRAGMENT and self.o.layout == ops.LAYOUT_FRAG16
                and self.nH // self.nKV <= 16 and getattr(ctx, "fragment_activations", False)):
            splits = ops.decode_attention_splits(T, self.nKV, ctx.max_context, self.window)
            slices = ops.linear_parts_slices(T, self.o.n, self.nH, self.d, splits) if splits > 1 else 0
            if slices > 0:
                parts, _ = ops.attention_decode(q, cache.k, cache.v, None, ctx.context_lens, cache.block_table,
                                                num_heads=self.nH, max_context=ctx.max_context, scale=self.scale,
                                                softcap=self.softcap, window=self.window, splits=splits)
                y = torch.empty((slices, T, self.o.n), dtype=torch.float32, device=q.device)
                ops.linear_parts(parts, splits, self.o.weight, y, num_heads=self.nH, head_dim=self.d)
                return y if slices > 1 else y[0]
        # The matrix-core kernels' output goes to the output projection in fragment order.
        frag = (getattr(ctx, "fragment_activations", False) and self.kv_layout == ops.KV_FRAGMENT
                and self.o.accepts_fragment_input and FragmentActs.possible(self.precision, T, self.q_dim))
        out = FragmentActs.empty(T, self.q_dim, q.device) if frag else torch.empty_like(q)
        ops.attention(q, cache.k, cache.v, out.data if frag else out, ctx, cache.block_table, num_heads=self.nH,
                      scale=self.scale, softcap=self.softcap, window=self.window, full_precision=self.precision.full,
                      kv_layout=self.kv_layout, out_layout=ops.LAYOUT_FRAG16 if frag else ops.LAYOUT_ROW,
                      bias_slopes=self._slopes)
        return self.o(out, torch.float32, allow_partials=True)
