"""The cache's bookkeeping and the generation loop's decisions (no GPU)."""
import random

import pytest
import torch

from alice_llm_amd.cache import Cache, CacheError, SlotTable
from alice_llm_amd.engine.generate import Generator, plan_batches
from alice_llm_amd.parts import CacheNeed, KVNeed, StateNeed
from alice_llm_amd.sampling import uniform


def needs(window=8):
    return [CacheNeed(kv=KVNeed(1, 16, window)), CacheNeed(kv=KVNeed(1, 16, None)), CacheNeed(kv=KVNeed(1, 16, window)), None]


def make(max_tokens=640, window=8, **kw):
    return Cache(needs(window), max_tokens=max_tokens, dtype=torch.float32, device="cpu", allocate=False, **kw)


def test_slot_table():
    t = SlotTable(3)
    a, b, c = t.take(), t.take(), t.take()
    assert sorted([a, b, c]) == [0, 1, 2] and t.n_free() == 0
    with pytest.raises(CacheError, match="all 3 slots"):
        t.take()
    t.give_back(b)
    with pytest.raises(CacheError, match="freed twice"):
        t.give_back(b)
    assert t.take() == b and t.length(b) == 0
    t.advance(a, 5)
    assert t.length(a) == 5 and t.held() == [0, 1, 2]
    with pytest.raises(CacheError):
        t.length(7)


def test_groups_by_need():
    c = make()
    assert [g.layers for g in c.groups] == [[0, 2], [1]] and [g.need.window for g in c.groups] == [8, None]
    assert c.max_tokens == 640 and c.groups[0].n_pages == 10


def test_pages_grow_trim_and_return():
    c = make(max_tokens=640, window=70)
    s = c.open()
    c.reserve([s], [200]); c.commit([s], [200])
    win, glob = c.groups
    assert len([p for p in glob.table(s) if p >= 0]) == 4
    # next query at 200 reads keys 131..200: pages 0 and 1 (positions 0..127) are out of reach
    assert [p >= 0 for p in win.table(s)] == [False, False, True, True]
    assert win.n_free() == 8 and glob.n_free() == 6
    c.check_consistent()
    c.reserve([s], [1]); c.commit([s], [1])
    assert c.length(s) == 201 and len(win.table(s)) == 4
    rows = c.block_table_rows(0, [s], 6)
    assert rows[0][:2] == [0, 0] and rows[0][4:] == [0, 0] and all(p > 0 for p in rows[0][2:4])
    c.close(s)
    assert win.n_free() == 10 and glob.n_free() == 10
    with pytest.raises(CacheError):
        c.close(s)
    c.check_consistent()


def test_capacity_error_before_any_change():
    c = make(max_tokens=256)
    a, b = c.open(), c.open()
    c.reserve([a, b], [100, 60]); c.commit([a, b], [100, 60])          # 2 + 1 pages of 4
    before = ([list(g.table(a)) for g in c.groups], [g.n_free() for g in c.groups])
    with pytest.raises(CacheError, match="cache is full"):
        c.reserve([a, b], [1, 100])                                      # b would need 2 more, 1 is free
    assert ([list(g.table(a)) for g in c.groups], [g.n_free() for g in c.groups]) == before
    with pytest.raises(CacheError, match="twice"):
        c.reserve([a, a], [1, 1])
    c.check_consistent()


def test_random_traffic_loses_nothing():
    rng = random.Random(0)
    c = make(max_tokens=64 * 40, window=100, max_seqs=6)
    live = {}
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and c.slots.n_free():
            live[c.open()] = 0
        elif op < 0.45 and live:
            s = rng.choice(list(live)); c.close(s); del live[s]
        elif live:
            ss = rng.sample(list(live), rng.randint(1, len(live)))
            ns = [rng.choice([1, 1, 1, 7, 64, 130]) for _ in ss]
            try:
                c.reserve(ss, ns)
            except CacheError:
                continue
            c.commit(ss, ns)
            for s, n in zip(ss, ns):
                live[s] += n
        c.check_consistent()
        assert all(c.length(s) == n for s, n in live.items())
    for s in list(live):
        c.close(s)
    c.check_consistent()
    assert all(g.n_free() == g.n_pages for g in c.groups) and c.slots.n_free() == 6


def test_state_region_is_zeroed_on_open():
    # two tensors of different shape and dtype for one run of the schedule, a row per slot and a spare row
    need = CacheNeed(state=(StateNeed("tail", (3, 2)), StateNeed("matrix", (4,), torch.float64)))
    c = Cache([need, None, CacheNeed(state=StateNeed("s", (1,)))], max_tokens=128, dtype=torch.float32, device="cpu", max_seqs=2)
    assert sorted(c.state) == [0, 2] and not c.groups and c.spare_slot == 2
    assert c.state[0]["tail"].shape == (3, 3, 2) and c.state[0]["matrix"].dtype == torch.float64
    s = c.open(); c.state[0]["tail"][s] += 5; c.state[0]["matrix"][s] -= 1; c.close(s)
    s2 = c.open()
    assert s2 == s and all(float(t[s2].abs().sum()) == 0.0 for t in c.state[0].values())
    view = c.view(0, [])
    assert set(view.state) == {"tail", "matrix"} and c.view(1, []).state == {}
    with pytest.raises(ValueError, match="distinct names"):
        CacheNeed(state=(StateNeed("a", (1,)), StateNeed("a", (2,))))


def test_page_size_is_the_caches_and_parts_can_insist_on_theirs():
    c = Cache(needs(), max_tokens=100, dtype=torch.float32, device="cpu", allocate=False, page_size=16)
    assert c.page_size == 16 and c.max_tokens == 112
    s = c.open(); c.reserve([s], [40]); c.commit([s], [40])
    assert len(c.groups[1].table(s)) == 3
    with pytest.raises(CacheError, match="pages of 64"):
        Cache([CacheNeed(kv=KVNeed(1, 16, None, page_size=64))], max_tokens=100, dtype=torch.float32, device="cpu",
              allocate=False, page_size=16)
    # keys and values of different head sizes get storage of their own shapes
    c = Cache([CacheNeed(kv=KVNeed(2, 16, None, value_head_dim=8))], max_tokens=64, dtype=torch.float32, device="cpu")
    assert c.groups[0].k.shape == (1, 2, 2, 64, 16) and c.groups[0].v.shape == (1, 2, 2, 64, 8)


# ------------------------------------------------------------------ the loop
class FakeEngine:
    """Scripted logits: token = (last token fed + 1) mod V for every sequence; records slot traffic."""

    def __init__(self, V=16, max_tokens=64 * 8, n_slots=4, max_positions=None, page_size=64):
        self.V = V
        if max_positions is not None:
            self.max_positions = max_positions
        self.cache = make(max_tokens=max_tokens, max_seqs=n_slots, page_size=page_size)
        self.opened, self.closed, self.steps = [], [], []

    def open(self, n):
        s = [self.cache.open() for _ in range(n)]
        self.opened += s
        return s

    def close(self, slots):
        for s in slots:
            self.cache.close(s)
        self.closed += list(slots)

    def step(self, slots, tokens, want):
        self.cache.reserve(slots, [len(t) for t in tokens]); self.cache.commit(slots, [len(t) for t in tokens])
        self.steps.append((list(slots), [len(t) for t in tokens]))
        rows = [i for i in range(len(slots)) if want == "last" or (not isinstance(want, str) and want[i])]
        assert want == "last" or all(want[i] == [len(tokens[i]) - 1] for i in rows)    # the loop asks for last rows only
        out = torch.zeros(len(rows), self.V)
        for r, i in enumerate(rows):
            out[r, (tokens[i][-1] + 1) % self.V] = 1.0
        return out


def argmax_sampler(logits, requests, draws):
    return logits.argmax(-1)


def test_plan_batches():
    assert plan_batches([5, 12, 17, 100], [8] * 4, max_batch=2, capacity_tokens=256, max_slots=4, page=64) == [[0, 1], [2, 3]]
    assert plan_batches([60, 60, 60], [10] * 3, max_batch=None, capacity_tokens=256, max_slots=8, page=64) == [[0, 1], [2]]
    # the page size is the cache's: with pages of 16 the same three requests (69 tokens -> 80 each) fit together
    assert plan_batches([60, 60, 60], [10] * 3, max_batch=None, capacity_tokens=256, max_slots=8, page=16) == [[0, 1, 2]]
    # the last token drawn is never fed back: 60 + 5 - 1 = 64 tokens are one page
    assert plan_batches([60, 60], [5, 5], max_batch=None, capacity_tokens=128, max_slots=8, page=64) == [[0, 1]]
    with pytest.raises(ValueError, match="request 1"):
        plan_batches([5, 300], [8, 8], max_batch=4, capacity_tokens=256, max_slots=4, page=64)


def test_plan_prompt_steps():
    from alice_llm_amd.engine.generate import plan_prompt_steps
    assert plan_prompt_steps([5, 12, 17], None) == [[(0, 0, 5), (1, 0, 12), (2, 0, 17)]]
    assert plan_prompt_steps([5, 12, 17], 100) == [[(0, 0, 5), (1, 0, 12), (2, 0, 17)]]
    # every step but the last is full; a prompt goes on where the step before left it
    assert plan_prompt_steps([5, 12, 17], 7) == [[(0, 0, 5), (1, 0, 2)], [(1, 2, 7)], [(1, 9, 3), (2, 0, 4)], [(2, 4, 7)], [(2, 11, 6)]]
    assert plan_prompt_steps([3, 3], 3) == [[(0, 0, 3)], [(1, 0, 3)]]
    assert plan_prompt_steps([4], 1) == [[(0, i, 1)] for i in range(4)]
    for lens, budget in (([6000] * 8, 16384), ([1, 70, 64, 129, 2], 64), ([9], 2)):
        steps = plan_prompt_steps(lens, budget)
        assert all(sum(n for _, _, n in st) == budget for st in steps[:-1]) and 0 < sum(n for _, _, n in steps[-1]) <= budget
        assert all(len({i for i, _, _ in st}) == len(st) for st in steps)              # a sequence once per step
        at = [0] * len(lens)
        for st in steps:
            for i, a, n in st:
                assert a == at[i] and n > 0
                at[i] += n
        assert at == lens
    with pytest.raises(ValueError):
        plan_prompt_steps([3], 0)


def test_the_loop_cuts_prompts_into_steps_of_its_budget():
    """Prompts that hold more tokens than a step's budget run in several steps, a long one in pieces; what the loop
    decides afterwards is what it decides with everything in one step."""
    prompts = [[1, 2, 3, 4, 5, 6, 7, 8, 9], [7], [4, 5, 6, 7, 8], [12, 13]]
    caps = [3, 4, 2, 5]
    runs = {}
    for budget in (None, 64, 7, 4, 1):
        eng = FakeEngineAhead(n_slots=4)
        res = Generator(eng, stop_token_ids=[], sampler=argmax_sampler, max_step_tokens=budget).run(prompts, caps)
        runs[budget] = [r.tokens for r in res]
        n_prompt_steps = len(plan_prompt_steps_of(budget, prompts))
        assert n_prompt_steps == {None: 1, 64: 1, 7: 3, 4: 5, 1: 17}[budget]
        fed = [0] * 4
        for sl, ns in eng.steps[:n_prompt_steps]:
            assert sum(ns) <= (budget or 17)
            for s_, n in zip(sl, ns):
                fed[eng.opened.index(s_)] += n
        assert fed == [9, 1, 5, 2]
        assert eng.cache.slots.n_free() == 4
        eng.cache.check_consistent()
    assert all(r == runs[None] for r in runs.values()) and runs[None] == [[10, 11, 12], [8, 9, 10, 11], [9, 10], [14, 15, 0, 1, 2]]


def plan_prompt_steps_of(budget, prompts):
    from alice_llm_amd.engine.generate import plan_prompt_steps
    return plan_prompt_steps([len(p) for p in prompts], budget)


def test_requests_that_would_outgrow_the_positions():
    from alice_llm_amd.engine.generate import limit_caps
    assert limit_caps([5, 10, 3], [100, 2, 0], 12) == [8, 2, 0]       # 5 + 8 - 1 = 12 positions; small caps untouched
    with pytest.raises(ValueError, match="request 1.*13 tokens"):
        limit_caps([5, 13], [1, 1], 12)
    # in the loop: the long request ends with "length" at the last position, its batch mates are untouched, and
    # no step ever asks the engine for a position beyond the limit
    eng = FakeEngine(max_positions=12)
    res = Generator(eng, stop_token_ids=[], sampler=argmax_sampler).run([[1, 2, 3, 4, 5], [7], [9, 10]], [100, 3, 4])
    assert [len(r.tokens) for r in res] == [8, 3, 4] and [r.finish_reason for r in res] == ["length"] * 3
    assert res[0].tokens == [6, 7, 8, 9, 10, 11, 12, 13]
    assert max(sum(n for sl, ns in eng.steps for s, n in zip(sl, ns) if s == slot) for slot in range(3)) == 12
    assert eng.cache.slots.n_free() == 4
    # a prompt that is too long is refused before any slot is taken or any step runs
    eng = FakeEngine(max_positions=12)
    with pytest.raises(ValueError, match="request 2"):
        Generator(eng, sampler=argmax_sampler).run([[1], [2], list(range(13))], [2, 2, 2])
    assert eng.opened == [] and eng.steps == []


def test_loop_observer_sees_the_runs_own_steps():
    seen = []
    def observer(requests, positions, logits, tokens):
        seen.append((list(requests), list(positions), logits.argmax(-1).tolist(), list(tokens)))
    gen = Generator(FakeEngine(), stop_token_ids=[9], sampler=argmax_sampler, observer=observer)
    res = gen.run([[1, 2, 3], [7]], [3, 5])
    assert [r.tokens for r in res] == [[4, 5, 6], [8]]
    # the first step's logits belong to the prompts' last positions; the stop token is seen though not kept
    assert seen[0] == ([0, 1], [2, 0], [4, 8], [4, 8]) and seen[1] == ([0, 1], [3, 1], [5, 9], [5, 9])
    assert seen[2] == ([0], [4], [6], [6]) and len(seen) == 3


def test_loop_stop_tokens_caps_and_slot_reuse():
    eng = FakeEngine()
    gen = Generator(eng, stop_token_ids=[9], max_batch=2, sampler=argmax_sampler)
    prompts = [[1, 2, 3], [7], [4, 5], [12, 13, 14, 15], [2]]
    caps = [4, 10, 0, 3, 2]
    res = gen.run(prompts, caps)
    assert [r.tokens for r in res] == [[4, 5, 6, 7], [8], [], [0, 1, 2], [3, 4]]
    assert [r.finish_reason for r in res] == ["length", "stop", "length", "length", "length"]     # 9 is not appended
    assert [r.prompt_tokens for r in res] == [3, 1, 2, 4, 1]
    # first step of a batch brings whole prompts of unequal length, later steps one token each; the batch shrinks
    assert eng.steps[0] == ([0, 1], [3, 1]) and eng.steps[1][1] == [1, 1] and eng.steps[2] == ([0], [1])
    assert sorted(eng.opened) == sorted(eng.closed) and len(eng.opened) == 4       # cap 0 takes no slot
    assert set(eng.opened) <= {0, 1}                                                # later batches use the same slots again
    eng.cache.check_consistent()
    assert eng.cache.slots.n_free() == 4
    gen2 = Generator(FakeEngine(), stop_token_ids=[9], sampler=argmax_sampler, include_stop_token=True)
    assert gen2.run([[7]], [10])[0].tokens == [8, 9]


class FakeEngineAhead(FakeEngine):
    """The same, and it takes one token id per sequence as a tensor, as the GPU engine does: the loop then
    queues a step before it has seen the ids of the step before."""
    takes_device_tokens = True

    def step(self, slots, tokens, want):
        if isinstance(tokens, torch.Tensor):
            assert tokens.dim() == 1 and tokens.numel() == len(slots)
            self.from_tensor = getattr(self, "from_tensor", 0) + 1
            tokens = [[int(t)] for t in tokens]
        return super().step(slots, tokens, want)


def test_loop_one_step_ahead_decides_as_the_plain_loop_does():
    prompts = [[1, 2, 3], [7], [4, 5], [12, 13, 14, 15], [2], [6], [5]]
    caps = [4, 10, 0, 3, 2, 1, 9]
    runs = []
    for cls in (FakeEngine, FakeEngineAhead):
        eng = cls(n_slots=4)
        gen = Generator(eng, stop_token_ids=[9], max_batch=3, sampler=argmax_sampler)
        res = gen.run(prompts, caps)
        runs.append(([r.tokens for r in res], [r.finish_reason for r in res]))
        assert sorted(eng.opened) == sorted(eng.closed)                 # every slot given back, once
        assert len(set(eng.opened)) <= 3
        eng.cache.check_consistent()
        assert eng.cache.slots.n_free() == 4
    assert runs[0] == runs[1]
    assert runs[1][0] == [[4, 5, 6, 7], [8], [], [0, 1, 2], [3, 4], [7], [6, 7, 8]]
    assert runs[1][1] == ["length", "stop", "length", "length", "length", "length", "stop"]
    assert eng.from_tensor > 0
    # Request 1 draws the stop token 9 in its second step; by then the loop had queued it for a third, whose row is
    # dropped: one row more than the plain loop ran, in that step only.  Ends by a cap are never run past.
    plain, ahead = FakeEngine(n_slots=4), FakeEngineAhead(n_slots=4)
    for eng in (plain, ahead):
        Generator(eng, stop_token_ids=[9], sampler=argmax_sampler).run([[1, 2, 3], [7]], [4, 10])
    assert [len(s) for s, _ in plain.steps] == [2, 2, 1, 1]
    assert [len(s) for s, _ in ahead.steps] == [2, 2, 2, 1]
    # an observer sees every step as it is: the loop then waits for each
    seen = []
    eng = FakeEngineAhead()
    Generator(eng, stop_token_ids=[9], sampler=argmax_sampler,
              observer=lambda requests, positions, logits, tokens: seen.append(list(tokens))).run([[1, 2, 3], [7]], [3, 5])
    assert seen == [[4, 8], [5, 9], [6]] and not hasattr(eng, "from_tensor")


def test_loop_gives_slots_back_on_error():
    eng = FakeEngine(max_tokens=128)
    def bad_sampler(logits, requests, draws):
        raise RuntimeError("boom")
    with pytest.raises(RuntimeError):
        Generator(eng, sampler=bad_sampler).run([[1], [2]], [3, 3])
    assert eng.cache.slots.n_free() == 4
    eng.cache.check_consistent()


def test_uniform_stream_is_per_request():
    a = [uniform(7, 3, n) for n in range(5)]
    assert a == [uniform(7, 3, n) for n in range(5)] and all(0 <= u < 1 for u in a)
    assert a != [uniform(8, 3, n) for n in range(5)] and a != [uniform(7, 4, n) for n in range(5)]
