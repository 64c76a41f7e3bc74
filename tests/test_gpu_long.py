"""The regime that serving runs in: contexts past the real window of 4,096 with the pages behind it given back,
pieces of a prompt on a long cached prefix, decode batches of 16 to 130 through captured steps, and more
(batch, context) buckets than captured steps are kept.  All against the plain implementation, in both dtypes.

Random N(0, 0.02) weights would hide a key that is read one place too far: among thousands of keys with nearly
equal weights one more or less changes nothing that a tolerance sees.  The models here therefore carry a marker:
tokens whose keys every query scores far above all others (helpers.write_marker_model).  Markers
are placed so that the window's edge passes over them in a prompt piece, in single-token steps, and in a piece
that follows after pages were given back; the tests assert that the plain implementation with a window one key
longer differs there by far more than the tolerance, so a kernel that is off by one cannot pass.
"""
import os
import tempfile

import pytest
import torch

import alice_llm_amd as alice
from helpers import TOL, max_err, plain_model, random_tokens, write_marker_model

pytestmark = pytest.mark.gpu
_TMP = tempfile.TemporaryDirectory(prefix="alice_long_")
_COMMON = dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", hidden_activation="gelu_pytorch_tanh",
               tie_word_embeddings=True, eos_token_id=1, bos_token_id=2, rope_theta=10000.0,
               attn_logit_softcapping=50.0, final_logit_softcapping=30.0, rms_norm_eps=1e-6)
LONG = {
    # the real window and position limit, head size 128, layers sliding / global / sliding
    "w4096-d128": dict(_COMMON, num_hidden_layers=3, hidden_size=256, num_attention_heads=4, num_key_value_heads=2,
                       head_dim=128, intermediate_size=512, vocab_size=512, sliding_window=4096,
                       query_pre_attn_scalar=128, max_position_embeddings=8192),
    # head size 256 as in the 2B and 9B models, a window of 1,024
    "w1024-d256": dict(_COMMON, num_hidden_layers=2, hidden_size=192, num_attention_heads=2, num_key_value_heads=1,
                       head_dim=256, intermediate_size=384, vocab_size=300, sliding_window=1024,
                       query_pre_attn_scalar=256, max_position_embeddings=2048),
}
MARKERS = (7, 8, 9)  # the markers' token ids
_CASES = {}


def marker_model(name):
    """(folder, plain model, tokens, layout): a random model edited so that the marker's key stands out."""
    if name in _CASES:
        return _CASES[name]
    raw = dict(LONG[name])
    folder = os.path.join(_TMP.name, name)
    write_marker_model(folder, raw, seed=11, markers=MARKERS)
    W = raw["sliding_window"]
    # the sequence: a prompt, a second piece that crosses the window, single tokens, a third piece that starts after
    # pages were given back, single tokens again
    cuts = [0, W - 96, W + 504, W + 544, W + 644, W + 664]
    toks = [x if x not in MARKERS else x + 10 for x in random_tokens(raw["vocab_size"], cuts[-1], 5)]
    # the query at p sees the marker at m up to p = m + W - 1: the edge passes in the second piece, in the single
    # tokens and in the third piece
    edges = [W + 299, W + 524, W + 604]
    for p, m in zip(edges, MARKERS):
        toks[p - (W - 1)] = m
    plain = plain_model(folder, dense=True)
    _CASES[name] = (folder, plain, toks, cuts, edges, plain.forward(toks))
    return _CASES[name]


@pytest.mark.parametrize("name", list(LONG))
def test_the_markers_make_the_windows_edge_visible(name):
    folder, plain, toks, cuts, edges, ref = marker_model(name)
    wider = plain_model(folder, dense=True)
    wider.window = plain.window + 1                         # what a kernel that reads one key too many computes
    other = wider.forward(toks)
    for p in edges:
        assert (other[p] - ref[p]).abs().max() < 2e-3       # still inside the window: one ordinary key more
        assert (other[p + 1] - ref[p + 1]).abs().max() > 0.25, "the marker does not stand out"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(LONG))
def test_long_context_pieces_and_single_tokens_past_the_window(name, dtype):
    folder, plain, toks, cuts, edges, ref = marker_model(name)
    W = plain.window
    model = alice.load(folder, dtype=dtype)
    scale = max(1.0, float(ref.abs().max()))
    outs = {}
    for graphs in (True, False):
        eng = model.engine(seq_lens=[len(toks), 200], use_graphs=graphs)
        assert eng.use_graphs == graphs
        if not graphs:
            for g in eng.cache.groups:                      # stale contents: a read outside a sequence's keys shows
                g.k.fill_(1e30)
                g.v.fill_(-1e30)
        s = eng.open(1)
        got = []
        first = list(range(cuts[1] - 70, cuts[1]))          # the prompt's last rows
        got.append((first, eng.step(s, [toks[:cuts[1]]], [first])))
        got.append((range(cuts[1], cuts[2]), eng.step(s, [toks[cuts[1]:cuts[2]]], "all")))
        win = [g for g in eng.cache.groups if g.need.window is not None][0]
        assert sum(p < 0 for p in win.table(s[0])) >= 6     # pages behind the window were given back
        for p in range(cuts[2], cuts[3]):
            got.append(([p], eng.step(s, [[toks[p]]], "last").clone()))
        got.append((range(cuts[3], cuts[4]), eng.step(s, [toks[cuts[3]:cuts[4]]], "all")))
        for p in range(cuts[4], cuts[5]):
            got.append(([p], eng.step(s, [[toks[p]]], "last").clone()))
        assert sum(p >= 0 for p in win.table(s[0])) <= W // eng.page_size + 2
        eng.cache.check_consistent()
        eng.close(s)
        assert all(g.n_free() == g.n_pages for g in eng.cache.groups)
        rows = [p for r, _ in got for p in r]
        outs[graphs] = torch.cat([o for _, o in got])
        err = (outs[graphs].double().cpu() - ref[rows]).abs().max(dim=-1).values
        worst = int(err.argmax())
        assert float(err.max()) < TOL[dtype] * scale, (graphs, rows[worst], float(err.max()))
        del eng
    assert max_err(outs[True], outs[False]) < (1e-5 if dtype == "float32" else TOL[dtype]) * scale


# ------------------------------------------------------------------ large decode batches
from helpers import TINY_C, model_folder

WIDE_2B = dict(_COMMON, num_hidden_layers=2, hidden_size=2304, num_attention_heads=8, num_key_value_heads=4,
               head_dim=256, intermediate_size=9216, vocab_size=1000, sliding_window=40, query_pre_attn_scalar=256,
               max_position_embeddings=512)


def _batch(plain, n_seqs, seed, longest, most_new):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(1, longest + 1, (n_seqs,), generator=g).tolist()
    news = torch.randint(2, most_new + 1, (n_seqs,), generator=g).tolist()
    seqs = [random_tokens(plain.V, n + m, 1000 * seed + i) for i, (n, m) in enumerate(zip(lens, news))]
    return lens, seqs


def _run_batches(model, plain, sizes, dtype, longest, most_new):
    """Batches of unequal prompts one after another on one engine: the prompts in one step, then single tokens
    through captured steps while the batch shrinks; every logits row against the plain implementation."""
    eng = model.engine(seq_lens=[longest + most_new] * max(sizes), max_seqs=max(sizes))
    assert eng.use_graphs
    worst = 0.0
    for number, n_seqs in enumerate(sizes):
        lens, seqs = _batch(plain, n_seqs, 7 + number, longest, most_new)
        refs = [plain.forward(s) for s in seqs]
        scale = max(1.0, max(float(r.abs().max()) for r in refs))
        slots = eng.open(n_seqs)
        got = eng.step(slots, [s[:n] for s, n in zip(seqs, lens)], "last")
        worst = max(worst, max_err(got, torch.stack([r[n - 1] for r, n in zip(refs, lens)])) / (TOL[dtype] * scale))
        live, step = list(range(n_seqs)), 0
        buckets = set()
        while live:
            got = eng.step([slots[i] for i in live], [[seqs[i][lens[i] + step]] for i in live], "last")
            buckets.add(len(live))
            ref = torch.stack([refs[i][lens[i] + step] for i in live])
            err = max_err(got, ref) / (TOL[dtype] * scale)
            assert err < 1.0, (n_seqs, step, len(live), err)
            worst = max(worst, err)
            step += 1
            done = [i for i in live if lens[i] + step >= len(seqs[i])]
            eng.close([slots[i] for i in done])
            live = [i for i in live if i not in done]
        assert max(buckets) == n_seqs and len(buckets) > 1      # the batch started whole and shrank
        eng.cache.check_consistent()
        assert eng.cache.slots.n_free() == max(sizes)
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_batches_of_16_to_130_on_a_tiny_model(dtype):
    folder = model_folder("tiny-c", "bfloat16")
    plain = plain_model(folder, dense=True)
    model = alice.load(folder, dtype=dtype)
    assert _run_batches(model, plain, [16, 64, 65, 130], dtype, longest=150, most_new=9) < 1.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_batches_of_64_and_65_at_the_2b_widths(dtype):
    folder = os.path.join(_TMP.name, "wide-2b")
    if not os.path.exists(folder):
        alice.write_random_model(folder, dict(WIDE_2B), seed=5)
    plain = plain_model(folder, dense=True)
    model = alice.load(folder, dtype=dtype)
    assert _run_batches(model, plain, [64, 65, 33], dtype, longest=50, most_new=5) < 1.0


def test_more_buckets_than_captured_steps_are_kept():
    """The least recently used captured step is dropped when a new bucket comes; a bucket that comes back is
    captured again.  Every step is compared with the plain implementation."""
    folder = model_folder("tiny-c", "bfloat16")
    plain = plain_model(folder, dense=True)
    model = alice.load(folder, dtype="bfloat16")
    from alice_llm_amd.engine.step import Engine
    eng = Engine(model.lm, max_tokens=64 * 40, max_seqs=16, max_graphs=3)
    seqs = [random_tokens(plain.V, 30 + 40, 300 + i) for i in range(16)]
    refs = [plain.forward(s) for s in seqs]
    slots = eng.open(16)
    eng.step(slots, [s[:30] for s in seqs], "none")
    pos = [30] * 16
    seen = []
    for step, n in enumerate([16, 7, 3, 2, 1, 16, 5, 1, 9, 2, 16, 3]):     # buckets 16 8 4 2 1 16 8 1 16 2 16 4
        rows = list(range(n))
        got = eng.step([slots[i] for i in rows], [[seqs[i][pos[i]]] for i in rows], "last")
        ref = torch.stack([refs[i][pos[i]] for i in rows])
        assert max_err(got, ref) < TOL["bfloat16"] * max(1.0, float(ref.abs().max())), (step, n)
        for i in rows:
            pos[i] += 1
        seen.append(set(eng._graphs))
        assert len(eng._graphs) <= 3
    assert len(set().union(*seen)) == 5 and (16, 512) not in seen[4] and (16, 512) in seen[5]    # dropped and captured again
    eng.close(slots)
    eng.cache.check_consistent()
