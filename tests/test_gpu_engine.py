"""The engine against the plain implementation, in 32-bit and in bfloat16: whole requests, the last 32
tokens one by one, unequal batches one after another on reused slots, long decoding, first tokens."""
import pytest
import torch

import alice_llm_amd as alice
import alice_llm_amd.engine.step as step_mod
from helpers import TINY, TOL, max_err, model_folder, plain_model, random_tokens

pytestmark = pytest.mark.gpu

CASES = [(n, d) for n in ("tiny-a", "tiny-b", "tiny-c", "tiny-d") for d in ("float32", "bfloat16")]
_MODELS = {}


def setup(name, dtype, stored="bfloat16", hot=1.0):
    key = (name, dtype, stored, hot)
    if key not in _MODELS:
        folder = model_folder(name, stored, hot)
        _MODELS[key] = (alice.load(folder, dtype=dtype), plain_model(folder))
    return _MODELS[key]


def tol(dtype, ref):
    return TOL[dtype] * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("name,dtype", CASES)
def test_each_request_alone_and_whole(name, dtype):
    model, plain = setup(name, dtype)
    eng = model.engine(max_tokens=512)
    for n, seed in ((1, 1), (2, 2), (9, 3), (64, 4), (65, 5), (200, 6)):
        toks = random_tokens(plain.V, n, seed)
        ref = plain.forward(toks)
        s = eng.open(1)
        got = eng.step(s, [toks], "all")
        eng.close(s)
        assert got.shape == ref.shape and got.dtype == torch.float32
        assert max_err(got, ref) < tol(dtype, ref), (n, max_err(got, ref))
    eng.cache.check_consistent()


@pytest.mark.parametrize("name,dtype", CASES)
def test_last_32_tokens_one_by_one(name, dtype):
    model, plain = setup(name, dtype)
    eng = model.engine(max_tokens=256)
    toks = random_tokens(plain.V, 150, 7)
    ref = plain.forward(toks)
    s = eng.open(1)
    got = [eng.step(s, [toks[:-32]], "all")]
    for t in toks[-32:]:
        got.append(eng.step(s, [[t]], "last"))
    eng.close(s)
    got = torch.cat(got)
    assert max_err(got, ref) < tol(dtype, ref)
    # the two ways of cutting agree with each other more closely than with the 64-bit oracle
    s = eng.open(1)
    whole = eng.step(s, [toks], "all")
    eng.close(s)
    assert max_err(got, whole) < (1e-5 if dtype == "float32" else tol(dtype, ref))


@pytest.mark.parametrize("name,dtype", CASES)
def test_unequal_batches_on_reused_slots(name, dtype):
    model, plain = setup(name, dtype)
    eng = model.engine(max_tokens=64 * 8, max_seqs=4)
    worst = 0.0
    for batch_no, lens in enumerate(((5, 12, 17), (3, 70, 14, 21), (130, 2))):
        seqs = [random_tokens(plain.V, n + 6 + 3 * i, 10 * batch_no + i) for i, n in enumerate(lens)]
        refs = [plain.forward(s) for s in seqs]
        slots = eng.open(len(seqs))
        assert set(slots) <= {0, 1, 2, 3}
        got = eng.step(slots, [s[:n] for s, n in zip(seqs, lens)], "all")      # prompts of unequal length, one step
        ref = torch.cat([r[:n] for r, n in zip(refs, lens)])
        worst = max(worst, max_err(got, ref) / tol(dtype, ref))
        live = list(range(len(seqs)))
        step = 0
        while live:                                                              # then one token each; shorter ones end earlier
            feed = [[seqs[i][lens[i] + step]] for i in live]
            got = eng.step([slots[i] for i in live], feed, "last")
            ref = torch.stack([refs[i][lens[i] + step] for i in live])
            worst = max(worst, max_err(got, ref) / tol(dtype, ref))
            step += 1
            done = [i for i in live if lens[i] + step >= len(seqs[i])]
            eng.close([slots[i] for i in done])
            live = [i for i in live if i not in done]
        eng.cache.check_consistent()
    assert worst < 1.0, worst
    assert eng.cache.slots.n_free() == 4


@pytest.mark.parametrize("name,dtype", [("tiny-a", "float32"), ("tiny-b", "bfloat16"), ("tiny-c", "bfloat16"), ("tiny-c", "float32")])
def test_long_decoding_across_pages_and_window(name, dtype):
    model, plain = setup(name, dtype)
    eng = model.engine(max_tokens=64 * 6, max_seqs=2)
    toks = random_tokens(plain.V, 300, 11)
    ref = plain.forward(toks)
    s = eng.open(2)                               # a second sequence keeps the batch mixed
    other = random_tokens(plain.V, 40, 12)
    got = [eng.step(s, [toks[:3], other], [[0, 1, 2], []])]
    got.append(eng.step([s[0]], [[toks[3]]], "last"))
    eng.close([s[1]])
    for t in toks[4:]:
        got.append(eng.step([s[0]], [[t]], "last"))
    got = torch.cat(got)
    assert max_err(got, ref) < tol(dtype, ref)
    win = [g for g in eng.cache.groups if g.need.window is not None][0]
    assert sum(p >= 0 for p in win.table(s[0])) < 5 - (win.need.window < 64)    # the window gave pages back
    eng.close([s[0]])
    eng.cache.check_consistent()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_hot_weights_reach_the_caps(dtype):
    # With N(0, 0.02) weights scores and logits stay far below the caps; this variant multiplies q, k and
    # the embedding so that both tanh stages bend the values.
    model, plain = setup("tiny-b", dtype, hot=12.0)
    toks = random_tokens(plain.V, 40, 13)
    ref = plain.forward(toks)
    uncapped = plain_model_without_caps(plain).forward(toks)
    assert (uncapped - ref).abs().max() > 0.5, "the caps do not bite in this variant"
    eng = model.engine(max_tokens=128)
    s = eng.open(1)
    got = eng.step(s, [toks], "all")
    eng.close(s)
    assert max_err(got, ref) < tol(dtype, ref) * (1 if dtype == "float32" else 3), max_err(got, ref)


def plain_model_without_caps(plain):
    import copy
    p = copy.copy(plain)
    p.cap_a = None
    p.cap_f = None
    return p


def linears_of(model):
    from alice_llm_amd.parts.linear import Linear
    return [(prefix + k, v) for prefix, part in model.lm.named_parts() for k, v in vars(part).items() if isinstance(v, Linear)]


def plain_with_rounded_matrices(folder, dense=False):
    """The plain implementation fed with the folder's tensors, its matrices rounded to bfloat16 (norm weights as stored)."""
    import json, os
    from safetensors.torch import load_file
    from plain.gemma2_plain import PlainGemma2
    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    tensors = {k: (v.to(torch.bfloat16) if v.dim() == 2 else v) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return PlainGemma2(config, tensors, dense=dense)


@pytest.mark.parametrize("name", ["tiny-b", "tiny-c"])
def test_stored_float32_is_rounded_once_on_the_bfloat16_path(name):
    """A folder stored in 32-bit: the 32-bit path keeps it, the bfloat16 path rounds every matrix to bfloat16 at load
    and runs it on the matrix-core kernels like a folder stored in bfloat16 (norm weights stay 32-bit); the run
    that keeps stored dtypes leaves the matrices 32-bit."""
    from alice_llm_amd.hip import ops
    folder = model_folder(name, "float32")
    model, plain = setup(name, "float32", stored="float32")
    assert all(l.weight.dtype == torch.float32 for _, l in linears_of(model))
    assert model.lm.layers[0].norms["pre_mixer"].weight.dtype == torch.float32
    mb, _ = setup(name, "bfloat16", stored="float32")
    assert len(linears_of(mb)) >= 4 * len(mb.lm.layers) + 1
    for where, l in linears_of(mb):
        assert l.weight.dtype == torch.bfloat16 and l.layout == ops.LAYOUT_FRAG16, where
    assert mb.lm.layers[0].norms["pre_mixer"].weight.dtype == torch.float32
    mk = alice.load(folder, dtype="bfloat16", keep_stored_dtype=True)
    assert all(l.weight.dtype == torch.float32 and l.layout == ops.LAYOUT_ROW for _, l in linears_of(mk))
    toks = random_tokens(plain.V, 133, 14)
    ref = plain.forward(toks)
    rounded = plain_with_rounded_matrices(folder).forward(toks)
    for m, d, r in ((model, "float32", ref), (mb, "bfloat16", rounded), (mk, "bfloat16", ref)):
        eng = m.engine(max_tokens=256)
        s = eng.open(1)
        got = [eng.step(s, [toks[:101]], "all")] + [eng.step(s, [[t]], "last") for t in toks[101:]]
        assert max_err(torch.cat(got), r) < tol(d, r), d


def test_step_argument_errors():
    model, plain = setup("tiny-a", "float32")
    eng = model.engine(max_tokens=128, max_seqs=2)
    s = eng.open(2)
    with pytest.raises(ValueError, match="vocabulary"):
        eng.step(s, [[1], [256]])
    with pytest.raises(ValueError, match="at least one token"):
        eng.step(s, [[1], []])
    with pytest.raises(ValueError, match="vocabulary"):
        eng.step(s, [[1, 2, -1], [3]])
    with pytest.raises(ValueError, match="want"):
        eng.step(s, [[1], [2]], "first")
    with pytest.raises(ValueError, match="want"):
        eng.step(s, [[1], [2]], [[0], [1]])
    assert eng.length(s[0]) == 0 and eng.length(s[1]) == 0        # nothing of a refused step stays
    with pytest.raises(alice.CacheError, match="full"):
        eng.step(s, [[1] * 70, [2] * 70])
    with pytest.raises(alice.CacheError, match="max_position"):
        eng.step([s[0]], [[1] * 600])
    assert eng.length(s[0]) == 0
    with pytest.raises(alice.CacheError, match="all 2 slots"):
        eng.open(1)
    eng.close(s)


@pytest.mark.parametrize("name,dtype", [("tiny-c", "bfloat16"), ("tiny-b", "float32")])
def test_captured_decode_steps_match_eager_on_every_replay(name, dtype):
    """Decode steps recorded into HIP graphs: every replay is compared with the same step run eagerly, with
    eager work (a prompt step of another batch, a shrinking batch, a new context bucket) between replays."""
    model, plain = setup(name, dtype)
    eager = model.engine(max_tokens=64 * 40, max_seqs=8, use_graphs=False)
    graph = model.engine(max_tokens=64 * 40, max_seqs=8, use_graphs=True)
    assert graph.use_graphs and not eager.use_graphs
    seqs = [random_tokens(plain.V, n, 50 + i) for i, n in enumerate((30, 75, 9, 520, 130))]
    lens = [10, 60, 3, 500, 100]
    se, sg = eager.open(5), graph.open(5)
    for eng, sl in ((eager, se), (graph, sg)):
        eng.step(sl, [s[:n] for s, n in zip(seqs, lens)], "none")
    live = list(range(5))
    step = 0
    while live:
        feed = [[seqs[i][lens[i] + step]] for i in live]
        a = eager.step([se[i] for i in live], feed, "last")
        b = graph.step([sg[i] for i in live], feed, "last").clone()
        assert a.shape == b.shape
        assert max_err(a, b) < (1e-5 if dtype == "float32" else 2e-2), (step, max_err(a, b))
        if step % 5 == 2:                                    # eager work between replays, on other slots
            extra = graph.open(1)
            graph.step(extra, [random_tokens(plain.V, 70, step)], "last")
            graph.close(extra)
        step += 1
        done = [i for i in live if lens[i] + step >= len(seqs[i])]
        for eng, sl in ((eager, se), (graph, sg)):
            eng.close([sl[i] for i in done])
        live = [i for i in live if i not in done]
    assert len(graph._graphs) >= 3            # batches of 5 (bucket 8), then fewer; a second context bucket past 512
    ref = plain.forward(seqs[3])
    s = graph.open(1)
    graph.step(s, [seqs[3][:500]], "none")
    got = torch.cat([graph.step(s, [[t]], "last").clone() for t in seqs[3][500:]])
    assert max_err(got, ref[500:]) < tol(dtype, ref)
    graph.cache.check_consistent()


def test_captured_prompt_pieces_on_a_long_prefix_past_the_window():
    """Recorded prompt steps in their second context bucket (keys up to 1,024) with the matrix-core kernels: pieces
    of 2 to 256 tokens on cached prefixes of more than 512 tokens, far enough past the window of 80 that the
    sliding layers' first pages were given back and their block-table entries point at the spare page.  The list of
    requests runs three times (seen once, recorded, replayed); every step against the eager engine and the plain
    implementation, the replay bit for bit against the recording pass."""
    model, plain = setup("tiny-c", "bfloat16")
    eager = model.engine(max_tokens=64 * 40, max_seqs=4, use_graphs=False)
    graph = model.engine(max_tokens=64 * 40, max_seqs=4, use_graphs=True)
    assert graph.capture_prompts
    win = [g for g in graph.cache.groups if g.need.window is not None][0]
    # (prefix lengths, then the pieces' lengths one step after another)
    rounds = [((530,), [(2,), (256,), (17,)]), ((600, 520), [(100, 30), (7, 9)]), ((700,), [(64,), (64,), (3,)]),
              ((515, 640, 580), [(5, 1, 60)])]
    recorded = {}
    for again in range(3):
        for r, (prefix, pieces) in enumerate(rounds):
            total = [n + sum(p[i] for p in pieces) for i, n in enumerate(prefix)]
            full = [random_tokens(plain.V, n, 700 + 10 * r + i) for i, n in enumerate(total)]
            refs = [plain.forward(s) for s in full]
            se, sg = eager.open(len(prefix)), graph.open(len(prefix))
            feed = [s[:n] for s, n in zip(full, prefix)]
            eager.step(se, feed, "none"); graph.step(sg, feed, "none")
            assert all(sum(p < 0 for p in win.table(s)) >= 6 for s in sg)          # pages behind the window are gone
            pos = list(prefix)
            outs = []
            for piece in pieces:
                feed = [s[p:p + n] for s, p, n in zip(full, pos, piece)]
                a, b = eager.step(se, feed, "last"), graph.step(sg, feed, "last")
                pos = [p + n for p, n in zip(pos, piece)]
                assert max_err(a, b) < 2e-2, (again, r, piece, max_err(a, b))
                for i in range(len(prefix)):
                    assert max_err(b[i], refs[i][pos[i] - 1]) < tol("bfloat16", refs[i]), (again, r, piece, i)
                outs.append(b.clone())
            if again == 1:
                recorded[r] = outs
            elif again == 2:
                assert all(torch.equal(x, y) for x, y in zip(recorded[r], outs)), r
            eager.close(se); graph.close(sg)
            graph.cache.check_consistent()
    keys = set(graph._prompt_graphs)
    assert all(k[2] == 1024 for k in keys) and {(1, 16, 1024, True), (1, 256, 1024, False), (1, 64, 1024, False),
                                                (2, 16, 1024, False), (2, 144, 1024, True), (3, 80, 1024, True)} <= keys
    assert all(g.graph is not None for g in graph._prompt_graphs.values())


@pytest.mark.parametrize("name,dtype", [("tiny-c", "bfloat16"), ("tiny-b", "float32"), ("tiny-a", "bfloat16")])
def test_captured_prompt_steps_match_eager_and_plain_on_every_replay(name, dtype, monkeypatch):
    """Steps of a few short prompts, or pieces of prompts, are recorded into HIP graphs as well (their token count
    rounded up, the tokens beyond the real ones on a sequence of the engine's own), from a shape's second sighting on.
    One graph serves every split of its tokens over its sequences: the same shape comes back with other splits, other
    slots and other cached prefixes, with eager work and decode steps between the replays, and every step is
    compared with the eager engine's and with the plain implementation.  The list of requests runs three times: the
    third pass (replays) must give the bits of the second (the recording pass), whatever the padding and the steps
    before left behind."""
    model, plain = setup(name, dtype)
    eager = model.engine(max_tokens=64 * 40, max_seqs=16, use_graphs=False)
    graph = model.engine(max_tokens=64 * 40, max_seqs=16, use_graphs=True)
    assert graph.capture_prompts and not eager.capture_prompts
    close = 1e-5 if dtype == "float32" else 2e-2
    # (prompt lengths, then lengths of a second piece or None): several share a shape (sequences, tokens rounded up)
    rounds = [((5, 9), None), ((9, 5), None), ((13, 1), None), ((1, 2), (12, 13)), ((20,), None), ((17,), (60,)),
              ((30, 1, 40), None), ((3, 3, 3, 3, 3, 3, 3, 3), None), ((100, 90), (20, 30)), ((2, 1) * 8, None)]
    recorded = {}
    for again in range(3):
        for r, (lens, more) in enumerate(rounds):
            full = [random_tokens(plain.V, n + (more[i] if more else 0) + 2, 900 + 10 * len(lens) + i) for i, n in enumerate(lens)]
            refs = [plain.forward(s) for s in full]
            se, sg = eager.open(len(lens)), graph.open(len(lens))
            if (r + again) % 2:
                sg = sg[::-1]
            pos = [0] * len(lens)
            outs = []
            for piece in ([lens] + ([more] if more else [])):
                feed = [s[p:p + n] for s, p, n in zip(full, pos, piece)]
                a = eager.step(se, feed, "last")
                b = graph.step(sg, feed, "last")
                pos = [p + n for p, n in zip(pos, piece)]
                assert max_err(a, b) < close, (again, r, piece, max_err(a, b))
                for i in range(len(lens)):
                    assert max_err(b[i], refs[i][pos[i] - 1]) < tol(dtype, refs[i]), (again, r, piece, i)
                outs.append(b.clone())
            for k in range(2):                               # then single tokens, through the captured decode steps
                feed = [[s[p]] for s, p in zip(full, pos)]
                a, b = eager.step(se, feed, "last"), graph.step(sg, feed, "last")
                pos = [p + 1 for p in pos]
                assert max_err(a, b) < close
                for i in range(len(lens)):
                    assert max_err(b[i], refs[i][pos[i] - 1]) < tol(dtype, refs[i])
            if again == 1:
                recorded[r] = outs
            elif again == 2:
                for x, y in zip(recorded[r], outs):
                    assert torch.equal(x, y), (r, lens)
            eager.close(se); graph.close(sg)
            graph.cache.check_consistent()
        if again == 0:                                       # only the shapes that came back within the list are recorded yet
            assert set(graph._prompt_graphs) == {(2, 16, 512, True), (1, 32, 512, True)}
    keys = set(graph._prompt_graphs)
    assert len(keys) < len(rounds) + 3 and all(g.graph is not None for g in graph._prompt_graphs.values())
    assert {(2, 16, 512, True), (8, 32, 512, True), (2, 64, 512, True), (2, 192, 512, True), (1, 64, 512, True), (16, 32, 512, True)} <= keys
    # other wanted rows and shapes seen once are not recorded
    n = len(keys)
    for again in range(3):                                   # a multiple of 16 tokens: no sequence of the engine's own
        toks = random_tokens(plain.V, 256 + 3, 3 + again)
        ref = plain.forward(toks)
        s = graph.open(1)
        assert max_err(graph.step(s, [toks[:256]], "last")[0], ref[255]) < tol(dtype, ref)
        assert max_err(graph.step(s, [toks[256:258]], "last")[0], ref[257]) < tol(dtype, ref)
        graph.close(s)
    assert set(graph._prompt_graphs) - keys == {(1, 256, 512, False), (1, 16, 512, True)}
    s = graph.open(1)
    for again in range(3):
        graph.step(s, [random_tokens(plain.V, 9, 4)], "all")
    graph.close(s)
    s = graph.open(1)
    graph.step(s, [random_tokens(plain.V, 100, 3)], "last")      # seen once
    graph.close(s)
    assert len(graph._prompt_graphs) == n + 2
    # the recorded steps kept hold a budget of tokens together (each keeps its activations): the oldest go
    monkeypatch.setattr(step_mod, "PROMPT_GRAPH_BUDGET", 300)
    for again in range(3):
        toks = random_tokens(plain.V, 200, 8 + again)
        ref = plain.forward(toks)
        s = graph.open(1)
        assert max_err(graph.step(s, [toks], "last")[0], ref[199]) < tol(dtype, ref)
        graph.close(s)
    assert (1, 208, 512, True) in graph._prompt_graphs and sum(k[1] for k in graph._prompt_graphs) <= 300
    assert len(graph._prompt_graphs) < n
    # beyond 256 tokens a step's kernels take longer than the host's launches: not recorded
    for again in range(3):
        s = graph.open(1)
        graph.step(s, [random_tokens(plain.V, 257, 3)], "last")
        graph.close(s)
    assert all(k[1] <= 256 for k in graph._prompt_graphs)


@pytest.mark.parametrize("name,dtype", [("tiny-c", "bfloat16"), ("tiny-b", "float32")])
@pytest.mark.parametrize("graphs", [True, False])
def test_token_ids_given_on_the_device(name, dtype, graphs):
    """One token id per sequence as a device tensor (what the sampling kernels return) gives the same bits as the
    same ids from the host, in captured and in eager steps, fed from the step before without the host seeing
    them; a batch that shrinks takes the ids of the rows that go on."""
    model, plain = setup(name, dtype)
    prompts = [random_tokens(plain.V, n, 70 + i) for i, n in enumerate((5, 40, 66))]
    a = model.engine(max_tokens=64 * 12, max_seqs=4, use_graphs=graphs)
    b = model.engine(max_tokens=64 * 12, max_seqs=4, use_graphs=graphs)
    sa, sb = a.open(3), b.open(3)
    ids_a = alice.sample(a.step(sa, prompts, "last"))
    ids_b = alice.sample(b.step(sb, prompts, "last"))
    assert torch.equal(ids_a, ids_b)
    seqs = [list(p) for p in prompts]
    for step in range(6):
        host = ids_a.tolist()
        for s, t in zip(seqs, host):
            s.append(t)
        la = a.step(sa, [[t] for t in host], "last")
        lb = b.step(sb, ids_b, "last")                       # never read on the host
        assert torch.equal(la, lb), step
        ids_a, ids_b = alice.sample(la), alice.sample(lb)
        if step == 2:                                        # the middle sequence ends
            a.close([sa.pop(1)]); b.close([sb.pop(1)]); seqs.pop(1)
            ids_a = ids_a[[0, 2]].contiguous()
            ids_b = ids_b[torch.tensor([0, 2], device=ids_b.device)]
    for s, la_row in zip(seqs, la):                          # and the ids were the greedy ones of the plain model
        ref = plain.forward(s)[-1]
        assert max_err(la_row, ref) < tol(dtype, ref)
    with pytest.raises(ValueError):
        b.step(sb, ids_b.long(), "last")
    with pytest.raises(ValueError):
        b.step(sb, ids_b.cpu(), "last")
    # an id outside the vocabulary cannot be refused by the host then: it embeds as zeros, and nothing is read out of bounds
    bad = torch.tensor([plain.V + 5, -1], dtype=torch.int32, device=ids_b.device)
    assert torch.isfinite(b.step(sb, bad, "last")).all()
    a.cache.check_consistent(); b.cache.check_consistent()


@pytest.mark.parametrize("name,dtype", [("tiny-b", "float32"), ("tiny-c", "bfloat16"), ("tiny-c", "float32")])
def test_stale_cache_contents_and_slot_order_change_nothing(name, dtype):
    """Pages are handed out again without being cleared.  Here every page of every pool is first filled with
    huge values: a kernel that read one position beyond a sequence's length, or before its window, would
    show it.  The same requests are then run in another slot order; logits are bitwise the same."""
    model, plain = setup(name, dtype)
    eng = model.engine(max_tokens=64 * 12, max_seqs=4, use_graphs=False)
    for g in eng.cache.groups:
        g.k.fill_(1e30)
        g.v.fill_(-1e30)
    seqs = [random_tokens(plain.V, n, 70 + i) for i, n in enumerate((100, 33, 65))]
    refs = [plain.forward(s) for s in seqs]

    def run(order):
        slots = eng.open(4)                       # one slot stays unused; its number shifts the others
        use = [slots[i] for i in order]
        a = eng.step(use, [s[:-2] for s in seqs], "all")
        b = eng.step(use, [[s[-2]] for s in seqs], "last")
        c = eng.step(use, [[s[-1]] for s in seqs], "last")
        eng.close(slots)
        return a, b, c

    a, b, c = run([0, 1, 2])
    ref_a = torch.cat([r[:-2] for r in refs])
    assert max_err(a, ref_a) < tol(dtype, ref_a)
    assert max_err(b, torch.stack([r[-2] for r in refs])) < tol(dtype, ref_a)
    assert max_err(c, torch.stack([r[-1] for r in refs])) < tol(dtype, ref_a)
    a2, b2, c2 = run([3, 0, 2])                   # other slots, other pages (the free list has been reshuffled)
    assert torch.equal(a, a2) and torch.equal(b, b2) and torch.equal(c, c2)
    a3, b3, c3 = run([3, 0, 2])                   # and run to run
    assert torch.equal(a2, a3) and torch.equal(c2, c3)
