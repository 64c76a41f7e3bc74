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

import numpy as np
import torch

from ..cache import Cache, CacheError, PAGE_SIZE
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
    # host copies, for parts that plan their launches on the host.  In a captured step (`captured`) they are
    # placeholders: a part that declares graph_safe reads the device arrays above instead.
    captured: bool = False
    new_lens: Sequence[int] = ()
    start_lens: Sequence[int] = ()
    slot_ids: Sequence[int] = ()
    # decode steps of at most 64 sequences in bfloat16: activations between the built-in parts travel in the
    # matrix-core kernels' fragment order (parts that do not declare support get plain tensors)
    fragment_activations: bool = False
    # every row is wanted, in order (a decode step's "last"): the final norm then needs no gather
    want_every_row: bool = False


Want = Union[str, Sequence[Sequence[int]]]


def _bucket(n: int) -> int:
    """Batch sizes that share a captured decode step: powers of two up to 64, then multiples of 64."""
    if n <= 64:
        b = 1
        while b < n:
            b *= 2
        return b
    return -(-n // 64) * 64


CONTEXT_BUCKET = 512        # captured decode steps are specialised to the context length rounded up to this
PROMPT_GRAPH_TOKENS = 256   # prompt steps of up to this many tokens are captured as well (beyond, the kernels take
                            # longer than the host's launches and a replay gains nothing),
PROMPT_GRAPH_SEQS = 16      # of at most this many sequences,
PROMPT_GRAPH_ROUND = 16     # their token count rounded up to a multiple of this;
PROMPT_GRAPH_BUDGET = 2048  # the captured steps kept hold this many tokens together (each keeps its activations)


class _Staging:
    """Pinned host buffers for the small integer arrays of a step, reused in turn; a buffer is written again
    only after the copy that last read it has run (pinned memory is allocated once, not per step)."""

    def __init__(self, n_buffers: int = 4):
        self.buffers = [None] * n_buffers
        self.events = [None] * n_buffers
        self.turn = 0

    def upload(self, values: np.ndarray, device) -> torch.Tensor:
        i = self.turn = (self.turn + 1) % len(self.buffers)
        if self.events[i] is not None:
            self.events[i].synchronize()
        n = len(values)
        if self.buffers[i] is None or self.buffers[i].numel() < n:
            self.buffers[i] = torch.empty(max(1024, 2 * n), dtype=torch.int32).pin_memory()
        host = self.buffers[i][:n]
        host.numpy()[:] = values
        out = torch.empty(n, dtype=torch.int32, device=device)
        out.copy_(host, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.events[i] = ev
        return out


class _DecodeGraph:
    """One captured decode step: its static integer inputs, its static logits, and pinned staging buffers."""

    def __init__(self, engine: "Engine", batch: int, context: int):
        self.batch, self.context = batch, context
        dev = engine.device
        self.width = -(-engine.max_positions // engine.cache.page_size)
        n_groups = len(engine.cache.groups)
        B = batch
        sizes = [B, B, B, B, B, B + 1, B] + [B * self.width] * n_groups
        self.offs = [0]
        for n in sizes:
            self.offs.append(self.offs[-1] + n)
        self.static = torch.zeros(self.offs[-1], dtype=torch.int32, device=dev)
        # The step's integers are kept in a host array that is updated in place (the block tables only when they
        # change) and copied through one of four pinned buffers; a pinned buffer is written again only after the
        # copy that last read it has run.  numpy views: a step writes a handful of short slices, and the time this
        # takes is time the GPU waits between two steps.
        self.shadow = np.zeros(self.offs[-1], dtype=np.int32)
        self.staging = [torch.zeros(self.offs[-1], dtype=torch.int32).pin_memory() for _ in range(4)]
        self.staging_np = [t.numpy() for t in self.staging]
        self.events = [torch.cuda.Event() for _ in range(4)]
        self.used = [False] * 4
        self.turn = 0
        part = lambda i: self.static[self.offs[i]:self.offs[i + 1]]
        self.block_tables = [part(7 + g).view(B, self.width) for g in range(n_groups)]
        self.ctx = StepContext(tokens=part(0), positions=part(1), seq_of_token=part(2), slots=part(3), want_rows=part(4),
                               cu_seqlens=part(5), context_lens=part(6), n_tokens=B, n_seqs=B, is_decode=True,
                               max_new=1, max_context=context, max_position=context - 1, new_lens=[1] * B,
                               captured=True, start_lens=[0] * B, slot_ids=[0] * B,
                               fragment_activations=engine.model.precision.act == torch.bfloat16,
                               want_every_row=True)
        o = self.offs
        self.shadow[o[2]:o[3]] = np.arange(B)                # constant parts
        self.shadow[o[4]:o[5]] = np.arange(B)
        self.shadow[o[5]:o[6]] = np.arange(B + 1)
        self.graph = None
        self.logits = None
        self.tables_version = None
        self.tables_slots = None

    def fill(self, engine: "Engine", slots, tokens, start) -> None:
        """Write this step's integers into a pinned buffer and queue its copy to the device."""
        B, n = self.batch, len(slots)
        o, sh = self.offs, self.shadow
        if self.tables_version != engine.cache.version or self.tables_slots != list(slots):
            for g in range(len(self.block_tables)):
                rows = engine.cache.block_table_rows(g, slots, self.width)
                tab = sh[o[7 + g]:o[8 + g]].reshape(B, self.width)
                tab[:n] = rows
                tab[n:] = 0                                  # padded rows: the spare page
            self.tables_version, self.tables_slots = engine.cache.version, list(slots)
        sh[o[0]:o[0] + n] = tokens
        sh[o[0] + n:o[1]] = 0
        sh[o[1]:o[1] + n] = start
        sh[o[1] + n:o[2]] = 0
        sh[o[3]:o[3] + n] = slots
        sh[o[3] + n:o[4]] = engine.cache.spare_slot          # padded rows: state of their own that nobody reads
        ctx_lens = sh[o[6]:o[7]]
        ctx_lens[:n] = start
        ctx_lens[:n] += 1
        ctx_lens[n:] = 1
        i = self.turn = (self.turn + 1) % len(self.staging)
        if self.used[i]:
            self.events[i].synchronize()                     # the copy that last used this buffer has run
        np.copyto(self.staging_np[i], sh)
        self.static.copy_(self.staging[i], non_blocking=True)
        self.events[i].record()
        self.used[i] = True


class _PromptGraph:
    """One captured step of a few prompts (or pieces of prompts): B sequences with T tokens in all, unequal.

    A short prompt's step is a few hundred launches of kernels that take microseconds; replayed from a graph it takes
    a third less time at 8 to 32 tokens and 4 % less at 128 (2B shape).  The graph is recorded for the token
    count rounded up to a multiple of 16 (the matrix products work in tiles of 16 tokens: the padding adds none);
    the tokens beyond the real ones, if any (`spare`), belong to one more sequence, of the engine's own, that lives
    on the cache's spare page, so that no kernel meets a sequence without tokens; what it computes is never read.
    Which tokens belong to which sequence is device data (cu_seqlens, seq_of_token, positions): the same graph
    serves any split of its tokens over B sequences."""

    def __init__(self, engine: "Engine", n_seqs: int, tokens: int, context: int, spare: bool):
        self.n_seqs, self.tokens, self.context, self.spare = n_seqs, tokens, context, spare
        dev = engine.device
        self.width = -(-engine.max_positions // engine.cache.page_size)
        n_groups = len(engine.cache.groups)
        B, T = n_seqs + (1 if spare else 0), tokens
        sizes = [T, T, T, B, B, B + 1, B] + [B * self.width] * n_groups
        self.offs = [0]
        for n in sizes:
            self.offs.append(self.offs[-1] + n)
        self.static = torch.zeros(self.offs[-1], dtype=torch.int32, device=dev)
        self.shadow = np.zeros(self.offs[-1], dtype=np.int32)
        self.staging = [torch.zeros(self.offs[-1], dtype=torch.int32).pin_memory() for _ in range(4)]
        self.staging_np = [t.numpy() for t in self.staging]
        self.events = [torch.cuda.Event() for _ in range(4)]
        self.used = [False] * 4
        self.turn = 0
        part = lambda i: self.static[self.offs[i]:self.offs[i + 1]]
        self.block_tables = [part(7 + g).view(B, self.width) for g in range(n_groups)]
        self.ctx = StepContext(tokens=part(0), positions=part(1), seq_of_token=part(2), slots=part(3), want_rows=part(4),
                               cu_seqlens=part(5), context_lens=part(6), n_tokens=T, n_seqs=B, is_decode=False,
                               max_new=T, max_context=context, max_position=context - 1, new_lens=[0] * B,
                               captured=True, start_lens=[0] * B, slot_ids=[0] * B,
                               fragment_activations=engine.model.precision.act == torch.bfloat16,
                               want_every_row=False)
        self.graph = None
        self.logits = None

    def fill(self, engine: "Engine", slots, new_tokens, start) -> None:
        B, T = self.n_seqs, self.tokens
        o, sh = self.offs, self.shadow
        n_new = [len(t) for t in new_tokens]
        used = sum(n_new)
        pad = T - used                                       # the engine's own sequence (none: pad == 0)
        assert (pad > 0) == self.spare and pad >= 0
        sh[o[0]:o[0] + used] = np.concatenate([np.asarray(seq, dtype=np.int64).reshape(-1) for seq in new_tokens])
        sh[o[1]:o[1] + used] = np.concatenate([np.arange(l, l + n) for l, n in zip(start, n_new)])
        sh[o[2]:o[2] + used] = np.repeat(np.arange(B), n_new)
        sh[o[3]:o[3] + B] = slots
        cu = np.concatenate(([0], np.cumsum(n_new)))
        sh[o[4]:o[4] + B] = cu[1:] - 1                       # the last token of each sequence
        sh[o[5]:o[5] + B + 1] = cu
        sh[o[6]:o[6] + B] = [l + n for l, n in zip(start, n_new)]
        if self.spare:
            sh[o[0] + used:o[1]] = 0
            sh[o[1] + used:o[2]] = np.arange(pad)
            sh[o[2] + used:o[3]] = B
            sh[o[3] + B] = engine.cache.spare_slot
            sh[o[4] + B] = T - 1
            sh[o[5] + B + 1] = T
            sh[o[6] + B] = pad
        rows = B + (1 if self.spare else 0)
        for g in range(len(self.block_tables)):
            tab = sh[o[7 + g]:o[8 + g]].reshape(rows, self.width)
            tab[:B] = engine.cache.block_table_rows(g, slots, self.width)
            if self.spare:
                tab[B] = 0                                   # the spare page
        i = self.turn = (self.turn + 1) % len(self.staging)
        if self.used[i]:
            self.events[i].synchronize()
        np.copyto(self.staging_np[i], sh)
        self.static.copy_(self.staging[i], non_blocking=True)
        self.events[i].record()
        self.used[i] = True


class Engine:
    """A model, its cache, and the step function over them."""

    takes_device_tokens = True      # step() accepts one token id per sequence as a device tensor

    def __init__(self, model: CausalLM, *, max_tokens: Optional[int] = None, seq_lens: Optional[Sequence[int]] = None,
                 max_seqs: Optional[int] = None, use_graphs: Optional[bool] = None, max_graphs: int = 24,
                 page_size: int = PAGE_SIZE):
        """The cache holds `max_tokens` tokens (each live sequence's count rounded up to whole pages), or, given
        `seq_lens` instead, room for sequences of these lengths at the same time."""
        self.model = model
        self.device = model.device
        ops.require_gpu()
        if (max_tokens is None) == (seq_lens is None):
            raise ValueError("give either max_tokens or seq_lens")
        if max_tokens is None:
            max_tokens = sum(-(-int(n) // page_size) * page_size for n in seq_lens)
            if max_seqs is None:
                max_seqs = len(seq_lens)
        # (the activation dtype is the pages' dtype unless a mixer's KVNeed names another)
        self.cache = Cache(model.cache_needs(), max_tokens=max_tokens, dtype=model.precision.act,
                           device=self.device, max_seqs=max_seqs, page_size=page_size)
        self.vocab_size = model.plan.vocab_size
        self.max_positions = model.plan.max_positions
        # Decode steps are captured into HIP graphs when every part says its launches can be recorded (parts
        # that loop on the host over sequences cannot).  A part with fixed-size state that says so indexes its
        # state with ctx.slots on the device; the padded rows of a captured step use the cache's spare slot.
        safe = model.graph_safe()
        self.use_graphs = safe if use_graphs is None else (use_graphs and safe)
        self._graphs = {}
        self._max_graphs = max_graphs
        # short prompt steps are captured too where the padding's positions exist and every part that keeps state
        # of its own says that it advances that state on the device in steps of several tokens
        self._prompt_graphs = {}
        self._prompt_seen = {}
        self.capture_prompts = (self.use_graphs and model.prompt_graph_safe()
                                and self.max_positions >= PROMPT_GRAPH_ROUND)
        self._staging = _Staging()

    # ------------------------------------------------------------------ sequences
    def open(self, n: int = 1) -> List[int]:
        return [self.cache.open() for _ in range(n)]

    def close(self, slots: Sequence[int]) -> None:
        for s in slots:
            self.cache.close(s)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    @property
    def page_size(self) -> int:
        return self.cache.page_size

    # ------------------------------------------------------------------ the step
    def step(self, slots: Sequence[int], new_tokens, want: Want = "last") -> torch.Tensor:
        """Run new_tokens[i] for the sequence in slots[i]; returns float32 logits [n_wanted, vocab].

        new_tokens: per sequence the list of its next token ids; or, for one token each, an int32 tensor [B] on
        the engine's device (what the sampling kernels return): the step is then queued without the host ever
        seeing the ids, so that a loop can queue the next step while this one runs.  An id outside the
        vocabulary, which the host cannot refuse then, embeds as a row of zeros.
        want: "last" (the last new token of each sequence), "all", "none", or per sequence a list of
        indices into its new tokens.  Rows come in the order of the sequences and of their lists.
        """
        B = len(slots)
        device_tokens = None
        if isinstance(new_tokens, torch.Tensor):
            if (new_tokens.dtype != torch.int32 or new_tokens.device != self.device or new_tokens.dim() != 1
                    or not new_tokens.is_contiguous()):
                raise ValueError(f"token ids given as a tensor must be contiguous int32 [sequences] on {self.device}")
            device_tokens = new_tokens
            new_tokens = [[0]] * new_tokens.numel()
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
        # the ids as one array (a prompt of thousands of tokens as Python lists costs the step a millisecond)
        flat = np.concatenate([np.asarray(seq, dtype=np.int64).reshape(-1) for seq in new_tokens])
        bad = flat[(flat < 0) | (flat >= self.vocab_size)]
        if bad.size:
            raise ValueError(f"token id {int(bad[0])} is outside the vocabulary of {self.vocab_size}")
        if not isinstance(want, str):
            want_lists = [list(w) for w in want]
            if len(want_lists) != B or any(not 0 <= i < n for w, n in zip(want_lists, n_new) for i in w):
                raise ValueError("want must give, per sequence, indices into its new tokens")
            if want_lists == [[n - 1] for n in n_new]:
                want = "last"                                  # said with indices: the same step
        elif want not in ("last", "all", "none"):
            raise ValueError('want is "last", "all", "none" or, per sequence, indices into its new tokens')
        self.cache.reserve(slots, n_new)                       # raises before any launch

        if self.use_graphs and want == "last" and max(n_new) == 1:
            logits = self._graph_step(slots, flat, start, device_tokens)
            self.cache.commit(slots, n_new)
            return logits
        if self.capture_prompts and want == "last" and B <= PROMPT_GRAPH_SEQS and len(flat) <= PROMPT_GRAPH_TOKENS:
            # recorded at a shape's second sighting: shapes that never come back cost nothing
            key = self._prompt_key(start, n_new)
            known = key in self._prompt_graphs
            if not known:
                self._prompt_seen[key] = self._prompt_seen.pop(key, 0) + 1
                if len(self._prompt_seen) > 512:
                    self._prompt_seen.pop(next(iter(self._prompt_seen)))
            if known or self._prompt_seen[key] >= 2:
                logits = self._prompt_graph_step(key, slots, new_tokens, start)
                self.cache.commit(slots, n_new)
                return logits

        cu = [0]
        for n in n_new:
            cu.append(cu[-1] + n)
        T = cu[-1]
        positions = np.concatenate([np.arange(l, l + n) for l, n in zip(start, n_new)])
        seq_of = np.repeat(np.arange(B), n_new)
        if want == "last":
            rows = [c - 1 for c in cu[1:]]
        elif want == "all":
            rows = np.arange(T)
        elif want == "none":
            rows = []
        else:
            rows = [cu[b] + i for b, w in enumerate(want_lists) for i in w]
        ctx_lens = [l + n for l, n in zip(start, n_new)]
        width = self.cache.table_width(slots)
        tables = [self.cache.block_table_rows(g, slots, width) for g in range(len(self.cache.groups))]

        # one host-to-device copy for all the small integer arrays of the step
        pieces = [flat, positions, seq_of, list(slots), rows, cu, ctx_lens] + [sum(t, []) for t in tables]
        packed = self._staging.upload(np.concatenate([np.asarray(p, dtype=np.int32).reshape(-1) for p in pieces]), self.device)
        offs = [0]
        for p in pieces:
            offs.append(offs[-1] + len(p))
        part = lambda i: packed[offs[i]:offs[i + 1]]
        block_tables = [part(7 + g).view(B, width) for g in range(len(tables))]
        if device_tokens is not None:
            part(0).copy_(device_tokens)
        ctx = StepContext(tokens=part(0), positions=part(1), seq_of_token=part(2), slots=part(3),
                          want_rows=part(4) if len(rows) else None, cu_seqlens=part(5), context_lens=part(6),
                          n_tokens=T, n_seqs=B, is_decode=all(n == 1 for n in n_new), max_new=max(n_new),
                          max_context=max(ctx_lens), max_position=max(ctx_lens) - 1,
                          new_lens=n_new, start_lens=start, slot_ids=list(slots),
                          fragment_activations=self.model.precision.act == torch.bfloat16,
                          want_every_row=len(rows) == T and (want == "all" or list(rows) == list(range(T))))
        logits = self.model.forward(ctx, self.cache, block_tables)
        self.cache.commit(slots, n_new)
        return logits

    # ------------------------------------------------------------------ captured prompt steps
    def _prompt_key(self, start, n_new):
        """(sequences, tokens rounded up, context bucket, whether the rounding left tokens for the engine's own sequence)"""
        used = sum(n_new)
        tokens = -(-used // PROMPT_GRAPH_ROUND) * PROMPT_GRAPH_ROUND
        reach = max(l + n for l, n in zip(start, n_new))
        context = min(self.max_positions, -(-reach // CONTEXT_BUCKET) * CONTEXT_BUCKET)
        return (len(n_new), tokens, context, tokens != used)

    def _prompt_graph_step(self, key, slots, new_tokens, start) -> torch.Tensor:
        """A few short prompts (or pieces) through a captured HIP graph, see _PromptGraph."""
        B = len(slots)
        g = self._prompt_graphs.get(key)
        if g is None:
            while self._prompt_graphs and (len(self._prompt_graphs) >= self._max_graphs or
                                           sum(k[1] for k in self._prompt_graphs) + key[1] > PROMPT_GRAPH_BUDGET):
                self._prompt_graphs.pop(next(iter(self._prompt_graphs)))
            g = self._prompt_graphs[key] = _PromptGraph(self, *key)
        else:
            self._prompt_graphs[key] = self._prompt_graphs.pop(key)
        g.fill(self, slots, new_tokens, start)
        if g.graph is None:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                first = self.model.forward(g.ctx, self.cache, g.block_tables)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                g.logits = self.model.forward(g.ctx, self.cache, g.block_tables)
            g.graph = graph
            return first[:B].clone()
        g.graph.replay()
        return g.logits[:B].clone()

    # ------------------------------------------------------------------ captured decode steps
    def _graph_step(self, slots, tokens, start, device_tokens=None) -> torch.Tensor:
        """One token per sequence through a captured HIP graph.  The batch is padded to a bucket size with
        rows that read and write only the cache's spare page; their logits are dropped."""
        B = len(slots)
        context = min(self.max_positions, -(-(max(start) + 1) // CONTEXT_BUCKET) * CONTEXT_BUCKET)
        key = (_bucket(B), context)
        g = self._graphs.get(key)
        if g is None:
            if len(self._graphs) >= self._max_graphs:
                self._graphs.pop(next(iter(self._graphs)))
            g = self._graphs[key] = _DecodeGraph(self, key[0], context)
        else:
            self._graphs[key] = self._graphs.pop(key)          # most recently used last
        g.fill(self, slots, tokens, start)
        if device_tokens is not None:
            g.ctx.tokens[:B].copy_(device_tokens)            # after the queued copy of the step's other integers
        if g.graph is None:
            # The first step of a bucket runs eagerly (which also warms up whatever the capture must not do for
            # the first time) and is then recorded without being run again: a part with state of its own would
            # otherwise advance that state twice.
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                first = self.model.forward(g.ctx, self.cache, g.block_tables)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                g.logits = self.model.forward(g.ctx, self.cache, g.block_tables)
            g.graph = graph
            return first[:B].clone()
        g.graph.replay()
        return g.logits[:B].clone()                          # the graph's own buffer is overwritten by its next replay
