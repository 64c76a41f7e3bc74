"""Parity in the regime that the benchmark runs: head sizes 256 and 128 with 8 query and 4 key heads, the real window
of 4,096 and 8,192 positions, batches of 8 and of 64 sequences with unequal contexts between 1,900 and 4,300 (and a
batch of 8 near 6,000), prompts through the generation loop's ragged steps of 16,384 tokens, then 40 single-token
steps, through captured steps and eagerly, in both dtypes.  Every logits row is compared with the plain
implementation, which runs in float64 on the GPU (a dense mask per head).

At these sizes single-token attention cuts a sequence's keys into 8 pieces at batch 8 and into one piece at
batch 64, whose four waves then walk 15 to 34 blocks of 32 keys each; the captured steps' block tables are 128
pages wide; and the
window's edge lies at another place in every sequence of a step.  The models carry markers
(helpers.write_marker_model): one at position 5 of every sequence, a far key that every query of a global layer
must find and that a sliding layer must lose at query 4,100 exactly, and one that the window's edge passes at
another single-token step in every sequence that is long enough.
"""
import os
import tempfile

import pytest
import torch

import alice_llm_amd as alice
from alice_llm_amd.hip import ops
from helpers import TOL, plain_model, random_tokens, write_marker_model

pytestmark = pytest.mark.gpu
_TMP = tempfile.TemporaryDirectory(prefix="alice_regime_")
_COMMON = dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", hidden_activation="gelu_pytorch_tanh",
               tie_word_embeddings=True, eos_token_id=1, bos_token_id=2, rope_theta=10000.0, num_hidden_layers=3,
               num_attention_heads=8, num_key_value_heads=4, attn_logit_softcapping=50.0, final_logit_softcapping=30.0,
               rms_norm_eps=1e-6, sliding_window=4096, max_position_embeddings=8192, vocab_size=512)
SHAPES = {
    "d256": dict(_COMMON, hidden_size=256, head_dim=256, intermediate_size=512, query_pre_attn_scalar=256),
    "d128": dict(_COMMON, hidden_size=192, head_dim=128, intermediate_size=448, query_pre_attn_scalar=144),
}
MARKERS = (7, 8, 9)
W, STEPS = 4096, 40
_CASES = {}


def _lengths(batch: str):
    """Prompt lengths of a batch; 40 single tokens follow each."""
    if batch == "8":
        return [1900, 2533, 3111, 3907, 4061, 4090, 4200, 4260]
    if batch == "8-long":
        return [5950, 5961, 6000, 5903, 6040, 5999, 6017, 5980]
    g = torch.Generator().manual_seed(21)
    lens = torch.randint(1900, 4261, (64,), generator=g).tolist()
    lens[3], lens[17], lens[40], lens[63] = 4062, 4099, 4096, 4260       # the far marker leaves the window while decoding
    return lens


def case(shape: str, batch: str):
    """(folder, sequences, prompt lengths, per sequence the reference logits at its prompt's last token and the
    40 that follow, the positions after which a marker has left the window)."""
    key = (shape, batch)
    if key in _CASES:
        return _CASES[key]
    folder = os.path.join(_TMP.name, shape)
    if not os.path.exists(folder):
        write_marker_model(folder, SHAPES[shape], seed=12, markers=MARKERS)
    V = SHAPES[shape]["vocab_size"]
    lens = _lengths(batch)
    seqs, edges = [], []
    for i, n in enumerate(lens):
        toks = [x if x not in MARKERS else x + 10 for x in random_tokens(V, n + STEPS, 100 * len(lens) + i)]
        toks[5] = MARKERS[0]                           # seen by queries up to position 5 + W - 1
        mine = [5 + W - 1] if n <= 5 + W - 1 < n + STEPS - 1 else []
        p = n + 3 + (7 * i) % (STEPS - 6)              # the last query that sees the second marker: another step in every sequence
        if p - (W - 1) > 5:
            toks[p - (W - 1)] = MARKERS[1]
            mine.append(p)
        seqs.append(toks)
        edges.append(mine)
    plain = plain_model(folder, dense=True, device="cuda")
    refs = [plain.forward(t)[n - 1:].float().cpu() for t, n in zip(seqs, lens)]
    # the markers do what they are for: with a window one key longer the row after an edge differs by far more than
    # any tolerance (checked on the sequences that have an edge, up to four of them)
    wider = plain_model(folder, dense=True, device="cuda")
    wider.window = W + 1
    checked = 0
    for t, n, r, mine in zip(seqs, lens, refs, edges):
        if mine and checked < 4:
            other = wider.forward(t)[n - 1:].float().cpu()
            for p in mine:
                assert (other[p + 1 - (n - 1)] - r[p + 1 - (n - 1)]).abs().max() > 0.25, "the marker does not stand out"
            checked += 1
    assert checked >= (1 if batch == "8-long" else 2)
    del plain, wider
    torch.cuda.empty_cache()
    _CASES[key] = (folder, seqs, lens, refs, edges)
    return _CASES[key]


def run_batch(eng, seqs, lens, refs, tol, name):
    """A batch from its prompts to 40 tokens each; returns all logits rows [sequences, 41, vocab]."""
    n_seqs = len(seqs)
    slots = eng.open(n_seqs)
    rows = [alice.run_prompt_steps(eng, slots, [s[:n] for s, n in zip(seqs, lens)]).cpu()]
    for step in range(STEPS):
        rows.append(eng.step(slots, [[s[n + step]] for s, n in zip(seqs, lens)], "last").cpu())
    got = torch.stack(rows, dim=1)
    ref = torch.stack(refs)
    err = (got.double() - ref.double()).abs().amax(dim=-1)             # [sequences, 41]
    scale = max(1.0, float(ref.abs().max()))
    worst = int(err.argmax())
    assert float(err.max()) < tol * scale, (name, "sequence", worst // (STEPS + 1), "row", worst % (STEPS + 1),
                                             float(err.max()), lens[worst // (STEPS + 1)])
    eng.cache.check_consistent()
    eng.close(slots)
    eng.cache.check_consistent()
    assert eng.cache.slots.n_free() == eng.cache.slots.n_slots and all(g.n_free() == g.n_pages for g in eng.cache.groups)
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", list(SHAPES))
def test_batches_of_8_and_64_at_contexts_up_to_4300(shape, dtype):
    model = alice.load(case(shape, "8")[0], dtype=dtype)
    nKV = SHAPES[shape]["num_key_value_heads"]
    # what the step's attention will do at these sizes (the bfloat16 path's split-key kernel)
    assert ops.decode_attention_splits(8, nKV, 4300, None) >= 7 and ops.decode_attention_splits(8, nKV, 4300, W) >= 7
    assert ops.decode_attention_splits(64, nKV, 4300, None) == 1 and ops.decode_attention_splits(64, nKV, 4300, W) == 1
    outs = {}
    for graphs in (True, False):
        eng = model.engine(seq_lens=[4352] * 64, max_seqs=64, use_graphs=graphs)
        assert eng.use_graphs == graphs
        if not graphs:
            for g in eng.cache.groups:                      # stale contents: a read outside a sequence's keys shows
                g.k.fill_(1e30)
                g.v.fill_(-1e30)
        for batch in ("8", "64", "8"):                      # one batch after another: slots and pages are used again
            folder, seqs, lens, refs, edges = case(shape, batch)
            got = run_batch(eng, seqs, lens, refs, TOL[dtype], (shape, dtype, batch, graphs))
            outs.setdefault((batch, graphs), got)
        if graphs:
            assert {k[0] for k in eng._graphs} == {8, 64}
        del eng
        torch.cuda.empty_cache()
    for batch in ("8", "64"):
        diff = float((outs[(batch, True)] - outs[(batch, False)]).abs().max())
        scale = max(1.0, float(outs[(batch, False)].abs().max()))
        assert diff < (1e-5 if dtype == "float32" else TOL[dtype]) * scale, (batch, diff)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_of_8_at_contexts_near_6000_with_the_window_biting_everywhere(dtype):
    folder, seqs, lens, refs, edges = case("d128", "8-long")
    assert all(len(e) == 1 for e in edges)                   # every sequence has a marker at its window's edge
    model = alice.load(folder, dtype=dtype)
    eng = model.engine(seq_lens=[max(lens) + STEPS] * 8, max_seqs=8)
    run_batch(eng, seqs, lens, refs, TOL[dtype], ("d128", dtype, "8-long"))
    win = [g for g in eng.cache.groups if g.need.window is not None][0]
    assert win.need.window == W
