"""Generation through the entry points: greedy tokens against the plain implementation, temperature
sampling reproducible by seed and independent of batch mates, the command line."""
import os
import subprocess
import sys

import pytest
import torch

import alice_llm_amd as alice
from helpers import model_folder, plain_model, random_tokens
from plain import gemma2_plain as P
from alice_llm_amd.sampling import uniform

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("name,lens,steps", [("tiny-a", (5, 12, 17), 8), ("tiny-b", (3, 9, 14, 21), 10)])
def test_greedy_generation_matches_plain(name, lens, steps):
    folder = model_folder(name, "bfloat16")
    plain = plain_model(folder)
    prompts = [random_tokens(plain.V, n, 30 + i) for i, n in enumerate(lens)]
    want = [plain.greedy(p, steps) for p in prompts]
    model = alice.load(folder, dtype="float32")
    res = model.generate(prompts, max_new_tokens=steps, stop_token_ids=[])
    assert [r.tokens for r in res] == want
    assert all(r.finish_reason == "length" and r.prompt_tokens == n for r, n in zip(res, lens))
    # one batch after another on two slots gives the same tokens
    res2 = model.generate(prompts, max_new_tokens=steps, stop_token_ids=[], max_batch=2)
    assert [r.tokens for r in res2] == want
    # a stop token ends its sequence early and is not part of the output
    stop = want[1][3]
    res3 = model.generate(prompts, max_new_tokens=steps, stop_token_ids=[stop])
    for r, w in zip(res3, want):
        cut = w.index(stop) if stop in w else len(w)
        assert r.tokens == w[:cut] and r.finish_reason == ("stop" if stop in w else "length")
    # bfloat16: every chosen token is at, or within rounding of, the plain model's maximum on the same prefix
    mb = alice.load(folder, dtype="bfloat16")
    for p, r in zip(prompts, mb.generate(prompts, max_new_tokens=steps, stop_token_ids=[])):
        seq = list(p)
        for tok in r.tokens:
            lg = plain.forward(seq)[-1]
            assert float(lg.max() - lg[tok]) < 0.03
            seq.append(tok)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompts_cut_into_steps_of_a_token_budget_give_the_same_tokens(dtype):
    """The loop runs a batch's prompts in ragged steps of at most max_step_tokens tokens: with budgets of 7 and 64
    (pieces that start and end inside pages and inside the window of 6, a piece of one token, a request that a step
    leaves out) and with none, greedy generation gives the same tokens, the plain implementation's."""
    folder = model_folder("tiny-b", "bfloat16")
    plain = plain_model(folder)
    prompts = [random_tokens(plain.V, n, 50 + i) for i, n in enumerate((3, 71, 14, 129, 1, 64))]
    model = alice.load(folder, dtype=dtype)
    steps_of = lambda budget: alice.plan_prompt_steps([len(p) for p in prompts], budget)
    assert [len(steps_of(b)) for b in (None, 64, 7)] == [1, 5, 41]
    assert any(n == 1 for st in steps_of(7) for _, _, n in st) and any(len(st) == 1 for st in steps_of(7))
    runs = {b: [r.tokens for r in model.generate(prompts, max_new_tokens=6, stop_token_ids=[], max_step_tokens=b)]
            for b in (None, 64, 7)}
    if dtype == "float32":
        assert runs[None] == [plain.greedy(p, 6) for p in prompts]
        assert runs[64] == runs[None] and runs[7] == runs[None]
    else:
        for b, run in runs.items():           # bfloat16: every chosen token within rounding of the plain maximum
            for p, toks in zip(prompts, run):
                seq = list(p)
                for tok in toks:
                    lg = plain.forward(seq)[-1]
                    assert float(lg.max() - lg[tok]) < 0.03, b
                    seq.append(tok)
    # the logits at the prompts' last tokens, through the loop's own prompt steps, against the plain implementation
    eng = model.engine(seq_lens=[len(p) for p in prompts])
    for b in (None, 64, 7):
        slots = eng.open(len(prompts))
        got = alice.run_prompt_steps(eng, slots, prompts, b)
        eng.close(slots)
        ref = torch.stack([plain.forward(p)[-1] for p in prompts])
        assert (got.double().cpu() - ref).abs().max() < (2e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max())), b
    eng.cache.check_consistent()


def test_generate_keeps_its_engine_between_calls():
    """Model.generate without an engine makes one and keeps it: a second call of the same shapes runs on the same
    cache and captures nothing new; a call that does not fit gets a larger engine."""
    folder = model_folder("tiny-c", "bfloat16")
    plain = plain_model(folder)
    model = alice.load(folder, dtype="bfloat16")
    prompts = [random_tokens(plain.V, n, 60 + i) for i, n in enumerate((9, 30, 17))]
    a = model.generate(prompts, max_new_tokens=8, stop_token_ids=[])
    eng = model._kept_engine
    assert eng is not None and eng.use_graphs and len(eng._graphs) >= 1
    graphs = dict(eng._graphs)
    prompt_graphs = dict(eng._prompt_graphs)
    b = model.generate(prompts, max_new_tokens=8, stop_token_ids=[])
    assert model._kept_engine is eng and [r.tokens for r in a] == [r.tokens for r in b]
    assert eng._graphs.keys() == graphs.keys() and all(eng._graphs[k] is g for k, g in graphs.items())
    c = model.generate(prompts[:2], max_new_tokens=5, stop_token_ids=[])            # smaller: fits
    assert model._kept_engine is eng and [len(r.tokens) for r in c] == [5, 5]
    d = model.generate(prompts + prompts, max_new_tokens=8, stop_token_ids=[])      # more sequences at once: a new engine
    assert model._kept_engine is not eng and [len(r.tokens) for r in d] == [8] * 6
    assert model._kept_engine.cache.slots.n_free() == 6
    model.release_engine()
    assert model._kept_engine is None


def test_temperature_sampling_is_reproducible_and_batch_independent():
    folder = model_folder("tiny-b", "bfloat16")
    plain = plain_model(folder)
    prompts = [random_tokens(plain.V, n, 40 + i) for i, n in enumerate((3, 9, 14, 21))]
    model = alice.load(folder, dtype="float32")
    kw = dict(max_new_tokens=10, temperature=0.8, seed=7, stop_token_ids=[])
    a = [r.tokens for r in model.generate(prompts, **kw)]
    assert a == [r.tokens for r in model.generate(prompts, **kw)]
    assert a != [r.tokens for r in model.generate(prompts, **dict(kw, seed=8))]
    assert a[:2] == [r.tokens for r in model.generate(prompts[:2], **kw)]            # same request index, other mates
    assert a == [r.tokens for r in model.generate(prompts, max_batch=3, **kw)]
    # against the plain sampler with the same uniform numbers (teacher-forced on the engine's own tokens)
    for r, (p, toks) in enumerate(zip(prompts, a)):
        seq = list(p)
        for n, tok in enumerate(toks):
            lg = plain.forward(seq)[-1]
            u = uniform(7, r, n)
            want = P.plain_sample(lg, 0.8, 0, 1.0, u)
            if want != tok:
                cdf = torch.cumsum(P.plain_softmax(lg / 0.8), 0)
                assert abs(float(cdf[min(tok, want)]) - u) < 1e-4
            seq.append(tok)
    greedy = [r.tokens for r in model.generate(prompts, max_new_tokens=10, temperature=0.0, stop_token_ids=[])]
    cold = [r.tokens for r in model.generate(prompts, max_new_tokens=10, temperature=1e-7, seed=3, stop_token_ids=[])]
    assert greedy == cold


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_loop_one_step_ahead_gives_what_the_waiting_loop_gives(dtype):
    """Generation queues step n + 1 from the ids on the device before the host has seen step n's; with an observer
    it waits for every step.  Both give the same tokens and reasons: with stop tokens drawn in the middle (the
    sequence has by then run one step ahead, and its slot goes to the next batch), unequal caps, several batches
    on few slots, greedy and with a temperature."""
    folder = model_folder("tiny-b", "bfloat16")
    plain = plain_model(folder)
    prompts = [random_tokens(plain.V, n, 90 + i) for i, n in enumerate((3, 9, 14, 21, 2, 33, 7))]
    model = alice.load(folder, dtype=dtype)
    free = model.generate(prompts, max_new_tokens=12, stop_token_ids=[])
    stops = [free[1].tokens[4], free[3].tokens[1], free[5].tokens[8]]
    caps = [12, 9, 1, 12, 5, 12, 2]
    seen = []
    for kw in (dict(), dict(temperature=0.9, seed=5, top_k=20)):
        runs = []
        for observer in (None, lambda requests, positions, logits, tokens: seen.append(len(tokens))):
            for max_batch in (None, 3):
                res = model.generate(prompts, max_new_tokens=caps, stop_token_ids=stops, max_batch=max_batch, observer=observer, **kw)
                runs.append([(r.tokens, r.finish_reason) for r in res])
        assert all(r == runs[0] for r in runs[1:])
        assert any(reason == "stop" for _, reason in runs[0]) and any(reason == "length" for _, reason in runs[0])
        assert all(len(t) <= c and not set(t) & set(stops) for (t, _), c in zip(runs[0], caps))
    assert seen


def test_command_line(tmp_path):
    folder = model_folder("tiny-a", "bfloat16")
    plain = plain_model(folder)
    prompts = [[5, 6, 7, 8], [100, 3]]
    want = [plain.greedy(p, 5) for p in prompts]
    cmd = [sys.executable, "-m", "alice_llm_amd.generate", "--model", folder, "--dtype", "float32", "--max-tokens", "5",
           "--temperature", "0", "--stop-ids", "", "--prompt-ids", "5,6,7,8", "--prompt-ids", "100,3", "--logits-dump", "2"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = proc.stdout.splitlines()
    assert f"[0] {','.join(map(str, want[0]))}  (length)" in lines and f"[1] {','.join(map(str, want[1]))}  (length)" in lines
    assert "Tokens: 10 generated, 6 prompt" in lines and any(l.startswith("Speed: ") and "tok/s" in l for l in lines)
    # the dump comes from the run's own steps: both requests, their first two generated positions, the token
    # the run's sampler drew there, and the plain implementation's five largest logits
    import json
    dumps = [json.loads(l) for l in proc.stderr.splitlines() if l.startswith("{")]
    assert [(d["request"], d["position"]) for d in dumps] == [(0, 3), (1, 1), (0, 4), (1, 2)]
    for d in dumps:
        seq = prompts[d["request"]] + want[d["request"]]
        lg = plain.forward(seq[:d["position"] + 1])[-1]
        top = torch.topk(lg, 5)
        assert d["token"] == seq[d["position"] + 1] == d["top5"][0][0]
        assert [t for t, _ in d["top5"]] == top.indices.tolist()
        assert max(abs(v - float(w)) for (_, v), w in zip(d["top5"], top.values)) < 2e-5
    # --dump-logits FILE: the same lines in a file, for every generated position
    path = tmp_path / "dump.jsonl"
    proc = subprocess.run(cmd[:-2] + ["--dump-logits", str(path)], capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert not [l for l in proc.stderr.splitlines() if l.startswith("{")]
    filed = [json.loads(l) for l in path.read_text().splitlines()]
    assert len(filed) == 10 and [d for d in filed if d["position"] in dict([(0, (3, 4)), (1, (1, 2))])[d["request"]]] == dumps


def test_logits_dump_follows_the_sampler_of_the_run():
    """With a temperature the dumped token is the one that was drawn and kept, which need not be the largest logit."""
    folder = model_folder("tiny-b", "bfloat16")
    model = alice.load(folder, dtype="float32")
    from alice_llm_amd.generate import _logits_dumper
    import contextlib, io, json
    err = io.StringIO()
    res = model.generate([[3, 4, 5], [9]], max_new_tokens=6, temperature=1.5, seed=3, stop_token_ids=[],
                         observer=_logits_dumper(4, err))
    dumps = [json.loads(l) for l in err.getvalue().splitlines()]
    assert len(dumps) == 8
    for r in (0, 1):
        mine = [d for d in dumps if d["request"] == r]
        assert [d["token"] for d in mine] == res[r].tokens[:4]
    assert any(d["token"] != d["top5"][0][0] for d in dumps)


def test_a_request_that_reaches_the_last_position_ends_alone():
    """One request of a batch would outgrow max_position_embeddings (512): it ends with "length" at the last
    position, its batch mates finish as they would alone, nothing is lost and no slot stays held."""
    folder = model_folder("tiny-a", "bfloat16")
    plain = plain_model(folder, dense=True)
    model = alice.load(folder, dtype="float32")
    eng = model.engine(seq_lens=[512, 64, 64], max_seqs=3)
    long_prompt, short = random_tokens(plain.V, 505, 80), random_tokens(plain.V, 9, 81)
    gen = alice.Generator(eng, stop_token_ids=[])
    res = gen.run([long_prompt, short, [5]], [40, 12, 3])
    assert [len(r.tokens) for r in res] == [8, 12, 3] and all(r.finish_reason == "length" for r in res)
    assert res[0].tokens == plain.greedy(long_prompt, 8) and res[1].tokens == plain.greedy(short, 12)
    assert eng.cache.slots.n_free() == 3
    eng.cache.check_consistent()
    with pytest.raises(ValueError, match="request 1.*513"):
        gen.run([[1, 2], [3] * 513], [4, 4])
    assert eng.cache.slots.n_free() == 3


def test_sample_and_step_of_the_python_surface():
    folder = model_folder("tiny-b", "bfloat16")
    plain = plain_model(folder)
    model = alice.load(folder, dtype="float32")
    eng = model.engine(max_tokens=128)
    toks = random_tokens(plain.V, 12, 90)
    s = eng.open(1)
    logits = model.step(eng, s, [toks], "all")                                  # the step function by its other name
    assert (logits.double().cpu() - plain.forward(toks)).abs().max() < 2e-5
    other = alice.load(folder, dtype="float32")
    with pytest.raises(ValueError, match="another model"):
        other.step(eng, s, [[1]])
    assert alice.sample(logits).tolist() == logits.argmax(-1).tolist()          # temperature 0: greedy, no u needed
    assert alice.sample(logits[3]).tolist() == [int(logits[3].argmax())]
    us = [uniform(5, 0, n) for n in range(12)]
    got = alice.sample(logits, temperature=0.9, top_k=7, top_p=0.8, u=us).tolist()
    for row, (g, u) in enumerate(zip(got, us)):
        want = P.plain_sample(logits[row].double().cpu(), 0.9, 7, 0.8, u)
        if g != want:                                                           # a draw within rounding of a boundary
            x = P.plain_top_p(P.plain_top_k(logits[row].double().cpu() / 0.9, 7), 0.8)
            cdf = torch.cumsum(P.plain_softmax(x), 0)
            assert abs(float(cdf[min(g, want)]) - u) < 1e-4
    with pytest.raises(ValueError, match="needs u"):
        alice.sample(logits, temperature=0.5)
    with pytest.raises(ValueError, match="one number"):
        alice.sample(logits, temperature=0.5, u=[0.1, 0.2])


def test_unexpected_tensors_are_an_error_or_a_warning(tmp_path):
    from safetensors.torch import load_file, save_file
    import shutil, warnings
    src = model_folder("tiny-a", "bfloat16")
    folder = str(tmp_path / "extra")
    shutil.copytree(src, folder)
    t = load_file(os.path.join(folder, "model.safetensors"))
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)
    save_file(t, os.path.join(folder, "model.safetensors"))
    with pytest.raises(alice.WeightError, match="unexpected \\(1\\): model.layers.0.self_attn.rotary_emb.inv_freq"):
        alice.load(folder, dtype="float32")
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        model = alice.load(folder, dtype="float32", strict=False)
    assert any(issubclass(x.category, alice.UnexpectedTensorsWarning) and "inv_freq" in str(x.message) for x in w)
    a, b = model.engine(64), alice.load(src, dtype="float32").engine(64)
    assert torch.equal(a.step(a.open(1), [[1, 2, 3]], "all"), b.step(b.open(1), [[1, 2, 3]], "all"))


def test_random_mode_matches_folder():
    raw = alice.preset("tiny-b")
    m1 = alice.load(raw, dtype="float32", random_seed=1)
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        alice.write_random_model(d, raw, 1)
        m2 = alice.load(d, dtype="float32")
        p = [[1, 2, 3, 4, 5]]
        e1, e2 = m1.engine(64), m2.engine(64)
        assert torch.equal(e1.step(e1.open(1), p, "all"), e2.step(e2.open(1), p, "all"))
