"""The generation loop above the step function: batches of unequal prompts, stop tokens, sequences
that end earlier, and as many batches one after another as there are requests.

A batch starts together: its prompts run in one ragged step, or, when they hold more tokens than a step's
budget, in several (a long prompt in pieces, logits asked for at its last piece only; the reference runs its
prompts request by request, llama3.rs:17783-17795); then every live sequence gets one token per
step.  A sequence ends when it draws a stop token (which is not part of its output, as in the
reference, llama3.rs:16137-16139) or reaches its own cap of new tokens (llama3.rs:17813-17835); it
leaves the batch at once and its slot goes back to the cache, where the next batch takes it.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

import torch


@dataclass
class GenerationResult:
    tokens: List[int]
    finish_reason: str              # "stop": a stop token was drawn; "length": the cap was reached
    prompt_tokens: int
    prefill_ms: float = 0.0         # of the batch the request ran in
    decode_ms: float = 0.0

    @property
    def tokens_generated(self) -> int:
        return len(self.tokens)


def limit_caps(prompt_lens: Sequence[int], caps: Sequence[int], max_positions: Optional[int]) -> List[int]:
    """Each request's cap of new tokens, cut so that the sequence never outgrows max_positions: a prompt of n
    tokens can draw max_positions - n + 1 tokens (the last one drawn is never fed back).  The reference ends
    such a sequence at its cap, not the whole call (llama3.rs:17813-17835).  A prompt that is itself longer than
    max_positions is an error, raised before anything runs, that names the request."""
    if max_positions is None:
        return [max(int(c), 0) for c in caps]
    out = []
    for i, (n, c) in enumerate(zip(prompt_lens, caps)):
        if n > max_positions:
            raise ValueError(f"request {i}: its prompt of {n} tokens is longer than the model's "
                             f"{max_positions} positions")
        out.append(max(0, min(int(c), max_positions - n + 1)))
    return out


def plan_batches(prompt_lens: Sequence[int], caps: Sequence[int], *, max_batch: Optional[int],
                 capacity_tokens: int, max_slots: int, page: int) -> List[List[int]]:
    """Split requests, in order, into batches that fit: at most max_batch (and max_slots) sequences,
    and room in the cache for every sequence at its longest, each rounded up to whole pages."""
    limit = min(max_batch or max_slots, max_slots)
    batches: List[List[int]] = []
    cur: List[int] = []
    used = 0
    for i, (n, c) in enumerate(zip(prompt_lens, caps)):
        need = -(-(n + max(c - 1, 0)) // page) * page         # the last token drawn is not fed back
        if need > capacity_tokens:
            raise ValueError(f"request {i} needs room for {need} tokens, the cache holds {capacity_tokens}")
        if cur and (len(cur) >= limit or used + need > capacity_tokens):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


MAX_STEP_TOKENS = 16384     # a prompt step's activations grow with its tokens (the gated product of the widest
                            # shape here takes 147 KB a token): 16,384 tokens keep them near 2 GB, and the
                            # matrix products are as fast per token from 8,192 tokens on


def plan_prompt_steps(prompt_lens: Sequence[int], max_step_tokens: Optional[int]) -> List[List[tuple]]:
    """Cut the prompts of a batch, in order, into steps of at most max_step_tokens tokens (None: one step).
    A step is a list of (index of the sequence in the batch, first token, number of tokens); a prompt that does
    not fit into what is left of a step goes on in the next one, so every step but the last is full.  A sequence
    appears at most once in a step, and its pieces come in consecutive steps."""
    if max_step_tokens is not None and max_step_tokens < 1:
        raise ValueError("a prompt step needs room for at least one token")
    budget = max_step_tokens or sum(prompt_lens) or 1
    steps: List[List[tuple]] = []
    cur: List[tuple] = []
    room = budget
    for i, n in enumerate(prompt_lens):
        at = 0
        while at < n:
            take = min(n - at, room)
            cur.append((i, at, take))
            at += take
            room -= take
            if room == 0:
                steps.append(cur)
                cur, room = [], budget
    if cur:
        steps.append(cur)
    return steps


def run_prompt_steps(engine, slots: Sequence[int], prompts: Sequence[Sequence[int]],
                     max_step_tokens: Optional[int] = MAX_STEP_TOKENS):
    """Run the prompts of sequences that start together, in as many ragged steps as the budget asks for; returns
    the logits at every prompt's last token, in the order of the sequences."""
    steps = plan_prompt_steps([len(p) for p in prompts], max_step_tokens)
    if len(steps) == 1:
        return engine.step(list(slots), [list(p) for p in prompts], "last")
    rows = []
    for step in steps:
        want = [[n - 1] if at + n == len(prompts[i]) else [] for i, at, n in step]
        logits = engine.step([slots[i] for i, _, _ in step], [list(prompts[i][at:at + n]) for i, at, n in step], want)
        if any(want):
            rows.append(logits)
    return rows[0] if len(rows) == 1 else torch.cat(rows)


class Generator:
    """Runs requests through an engine.  `engine` needs open(n), step(slots, tokens, want) and
    close(slots) and a cache with `max_tokens` and `slots.n_slots`; `sampler(logits, requests, draws)`
    returns one token id per row (anything with .tolist())."""

    def __init__(self, engine, *, temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, seed: int = 0,
                 stop_token_ids: Sequence[int] = (), max_batch: Optional[int] = None,
                 sampler: Optional[Callable] = None, include_stop_token: bool = False,
                 observer: Optional[Callable] = None, max_step_tokens: Optional[int] = MAX_STEP_TOKENS):
        """max_step_tokens: the most tokens of prompts that one step runs (None: a batch's prompts in one step).
        observer(requests, positions, logits, tokens), if given, is called after every step of every batch
        with the live requests' indices, the position each row's logits belong to, the step's float32 logits
        [rows, vocab] and the token ids drawn from them: what a logits dump of the real run needs."""
        self.engine = engine
        if sampler is None:
            from ..sampling import Sampler
            sampler = Sampler(temperature, top_k, top_p, seed)
        self.sampler = sampler
        self.stop = set(int(t) for t in stop_token_ids)
        self.max_batch = max_batch
        self.include_stop_token = include_stop_token
        self.observer = observer
        self.max_step_tokens = max_step_tokens
        plan_prompt_steps([], max_step_tokens)                   # refuses a budget below one token

    def run(self, prompts: Sequence[Sequence[int]], max_new_tokens: Sequence[int]) -> List[GenerationResult]:
        if len(prompts) != len(max_new_tokens):
            raise ValueError("one cap of new tokens per prompt")
        if any(len(p) == 0 for p in prompts):
            raise ValueError("every prompt needs at least one token")
        results: List[Optional[GenerationResult]] = [None] * len(prompts)
        cache = self.engine.cache
        lens = [len(p) for p in prompts]
        # everything that can be refused is refused here, before a slot is taken or a kernel runs
        caps = limit_caps(lens, max_new_tokens, getattr(self.engine, "max_positions", None))
        batches = plan_batches(lens, caps, max_batch=self.max_batch, capacity_tokens=cache.max_tokens,
                               max_slots=cache.slots.n_slots, page=cache.page_size)
        for batch in batches:
            self._run_batch(batch, prompts, caps, results)
        return results  # type: ignore[return-value]

    def _run_batch(self, batch, prompts, caps, results) -> None:
        """One batch from its prompts to its last token.  With an engine that takes token ids as a device tensor
        (and no observer to show every step to), the loop runs one step ahead of what it has seen: step n + 1 is
        queued, fed from the sampling kernel's output on the device, before the ids of step n have reached the
        host, so the GPU does not wait for the host between two steps.  Ends by a cap are known beforehand; a
        sequence that draws a stop token has by then been queued for one more step, whose result is dropped (its
        slot is given back at once: the pages it may hand to a later step are written by that step after this
        one)."""
        eng = self.engine
        out = {r: [] for r in batch}
        reason = {}
        live = [r for r in batch if caps[r] > 0]
        for r in batch:
            if caps[r] <= 0:
                reason[r] = "length"
        slots = dict(zip(live, eng.open(len(live))))
        ahead = self.observer is None and getattr(eng, "takes_device_tokens", False)
        t0 = time.perf_counter()
        prefill_ms = 0.0
        try:
            rows = list(live)                                # the requests of the step whose ids are on their way
            drawn = None                                     # that step's ids on the device and, later, on the host
            if rows:
                logits = run_prompt_steps(eng, [slots[r] for r in rows], [prompts[r] for r in rows], self.max_step_tokens)
                drawn = self._draw(logits, rows, out, 0)
            first = True
            while rows:
                queued = None
                alive = [r for r in rows if r not in reason]
                if ahead:
                    # the sequences that go on unless they draw a stop token now
                    nxt = [r for r in alive if len(out[r]) + 1 < caps[r]]
                    if nxt:
                        ids_dev = drawn[0]
                        if len(nxt) != len(rows):
                            pick = torch.tensor([rows.index(r) for r in nxt], dtype=torch.int64)
                            ids_dev = ids_dev[pick.to(ids_dev.device)]
                        logits = eng.step([slots[r] for r in nxt], ids_dev, "last")
                        queued = (nxt, self._draw(logits, nxt, out, 1))
                ids = drawn[1]()                             # waits for the step before the queued one only
                if first:
                    prefill_ms = (time.perf_counter() - t0) * 1e3
                    first = False
                if self.observer is not None:
                    self.observer(list(rows), [len(prompts[r]) + len(out[r]) - 1 for r in rows], drawn[2], ids)
                feed = []
                for r, tok in zip(rows, ids):
                    if r in reason:                          # ended a step ago: this row ran ahead for nothing
                        continue
                    tok = int(tok)
                    if tok in self.stop:
                        if self.include_stop_token:
                            out[r].append(tok)
                        reason[r] = "stop"
                    else:
                        out[r].append(tok)
                        if len(out[r]) >= caps[r]:
                            reason[r] = "length"
                    if r in reason:
                        eng.close([slots.pop(r)])            # the slot is free for the next batch at once
                    else:
                        feed.append((r, tok))
                if queued is not None:
                    rows, drawn = queued
                    if all(r in reason for r in rows):
                        rows = []
                elif feed:
                    rows = [r for r, _ in feed]
                    logits = eng.step([slots[r] for r in rows], [[tok] for _, tok in feed], "last")
                    drawn = self._draw(logits, rows, out, 0)
                else:
                    rows = []
        finally:
            if slots:
                eng.close(list(slots.values()))
        decode_ms = (time.perf_counter() - t0) * 1e3 - prefill_ms
        for r in batch:
            results[r] = GenerationResult(tokens=out[r], finish_reason=reason[r], prompt_tokens=len(prompts[r]),
                                          prefill_ms=prefill_ms, decode_ms=decode_ms)

    def _draw(self, logits, rows, out, pending: int):
        """Samples a step's rows (request r has drawn len(out[r]) + pending tokens before).  Returns the ids on
        the device, a function that gives them as a list once they have reached the host, and the logits."""
        ids = self.sampler(logits, rows, [len(out[r]) + pending for r in rows])
        if not (isinstance(ids, torch.Tensor) and ids.is_cuda):
            return ids, ids.tolist, logits
        host = torch.empty(ids.shape, dtype=ids.dtype, pin_memory=True)
        host.copy_(ids, non_blocking=True)
        done = torch.cuda.Event()
        done.record()

        def fetch():
            done.synchronize()
            return host.tolist()
        return ids, fetch, logits
