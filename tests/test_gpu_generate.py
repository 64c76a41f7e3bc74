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
    dumps = [l for l in proc.stderr.splitlines() if l.startswith("{")]
    assert len(dumps) == 2 and '"position": 3' in dumps[0] and f"[{want[0][0]}," in dumps[0].replace(" ", "").replace("[[", "[")


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
