"""The step function: a batch of sequences, each with its next tokens, run as one batch from the
cache, returning logits at the wanted places.

A step is either the first of its batch (every sequence brings its whole prompt, lengths unequal)
or a continuation (one token each); the same code also runs any number of new tokens on top of any
cached length, which is what cutting a prompt into pieces needs.  Tokens of all sequences are
concatenated without padding; positions continue from each slot's length.  The reference runs one
token of one sequence per call (llama3.rs:13496, position implicit in the cache cursor, 13682) and
loops over prompts and requests (llama3.rs:17783-17835).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Union

import torch

from ..cache import Cache, CacheError
from ..hip import ops
from .model import CausalLM


@dataclass
class StepContext:
    """Device-side description of a step, shared by all parts."""
    tokens: torch.Tensor            # int32 [T]
    positions: torch.Tensor         # int32 [T] absolute position of each token in its sequence
    seq_of_token: torch.Tensor      # int32 [T] index of the token's sequence within the step
    slots: torch.Tensor             # int32 [B] cache slot of each sequence (for fixed-size state)
    want_rows: Optional[torch.Tensor]   # int32 [n_out] rows of the step whose logits are wanted
    cu_seqlens: torch.Tensor        # int32 [B + 1] offsets of the sequences' tokens
    context_lens: torch.Tensor      # int32 [B] keys each sequence holds after the step
    n_tokens: int
    n_seqs: int
    is_decode: bool                 # every sequence brings exactly one token
    max_new: int                    # most new tokens of one sequence
    max_context: int                # most keys of one sequence after the step
    max_position: int               # largest position in the step
    # host copies, for parts that plan their launches
    new_lens: Sequence[int] = ()
    start_lens: Sequence[int] = ()
    slot_ids: Sequence[int] = ()


Want = Union[str, Sequence[Sequence[int]]]


class Engine:
    """A model, its cache, and the step function over them."""

    def __init__(self, model: CausalLM, *, max_tokens: int, max_seqs: Optional[int] = None):
        self.model = model
        self.device = model.device
        ops.require_gpu()
        self.cache = Cache(model.cache_needs(), max_tokens=max_tokens, dtype=model.precision.act,
                           device=self.device, max_seqs=max_seqs)
        self.vocab_size = model.plan.vocab_size
        self.max_positions = model.plan.max_positions

    # ------------------------------------------------------------------ sequences
    def open(self, n: int = 1) -> List[int]:
        return [self.cache.open() for _ in range(n)]

    def close(self, slots: Sequence[int]) -> None:
        for s in slots:
            self.cache.close(s)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # ------------------------------------------------------------------ the step
    def step(self, slots: Sequence[int], new_tokens: Sequence[Sequence[int]], want: Want = "last") -> torch.Tensor:
        """Run new_tokens[i] for the sequence in slots[i]; returns float32 logits [n_wanted, vocab].

        want: "last" (the last new token of each sequence), "all", "none", or per sequence a list of
        indices into its new tokens.  Rows come in the order of the sequences and of their lists.
        """
        B = len(slots)
        if B == 0 or len(new_tokens) != B:
            raise ValueError("a step needs at least one sequence and one token list per sequence")
        n_new = [len(t) for t in new_tokens]
        if min(n_new) < 1:
            raise ValueError("every sequence of a step brings at least one token")
        start = [self.cache.length(s) for s in slots]
        for s, l, n in zip(slots, start, n_new):
            if l + n > self.max_positions:
                raise CacheError(f"slot {s} would reach {l + n} tokens, beyond max_position_embeddings "
                                 f"{self.max_positions}")
        flat = [int(t) for seq in new_tokens for t in seq]
        bad = [t for t in flat if not 0 <= t < self.vocab_size]
        if bad:
            raise ValueError(f"token id {bad[0]} is outside the vocabulary of {self.vocab_size}")
        if want == "last":
            want_lists = [[n - 1] for n in n_new]
        elif want == "all":
            want_lists = [list(range(n)) for n in n_new]
        elif want == "none":
            want_lists = [[] for _ in n_new]
        else:
            want_lists = [list(w) for w in want]
            if len(want_lists) != B or any(not 0 <= i < n for w, n in zip(want_lists, n_new) for i in w):
                raise ValueError("want must give, per sequence, indices into its new tokens")
        self.cache.reserve(slots, n_new)                       # raises before any launch

        cu = [0]
        for n in n_new:
            cu.append(cu[-1] + n)
        T = cu[-1]
        positions = [l + i for l, n in zip(start, n_new) for i in range(n)]
        seq_of = [b for b, n in enumerate(n_new) for _ in range(n)]
        rows = [cu[b] + i for b, w in enumerate(want_lists) for i in w]
        ctx_lens = [l + n for l, n in zip(start, n_new)]
        width = self.cache.table_width(slots)
        tables = [self.cache.block_table_rows(g, slots, width) for g in range(len(self.cache.groups))]

        # one host-to-device copy for all the small integer arrays of the step
        pieces = [flat, positions, seq_of, list(slots), rows, cu, ctx_lens] + [sum(t, []) for t in tables]
        packed = torch.tensor(sum(pieces, []), dtype=torch.int32).pin_memory().to(self.device, non_blocking=True)
        offs = [0]
        for p in pieces:
            offs.append(offs[-1] + len(p))
        part = lambda i: packed[offs[i]:offs[i + 1]]
        block_tables = [part(7 + g).view(B, width) for g in range(len(tables))]
        ctx = StepContext(tokens=part(0), positions=part(1), seq_of_token=part(2), slots=part(3),
                          want_rows=part(4) if rows else None, cu_seqlens=part(5), context_lens=part(6),
                          n_tokens=T, n_seqs=B, is_decode=all(n == 1 for n in n_new), max_new=max(n_new),
                          max_context=max(ctx_lens), max_position=max(ctx_lens) - 1,
                          new_lens=n_new, start_lens=start, slot_ids=list(slots))
        logits = self.model.forward(ctx, self.cache, block_tables)
        self.cache.commit(slots, n_new)
        return logits
