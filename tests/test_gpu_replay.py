"""bin/trace_run as a user runs it: the same requests replayed whole, with the last 32 tokens one by
one, and in batches of unequal lengths one after another, in 32-bit and in bfloat16, all compared
with the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import TOL, model_folder, plain_model, random_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def round64(n):
    return -(-n // 64) * 64


def build_trace(requests):
    """Returns (lines, expectations, max_tokens); expectations: step -> list of (request, position)."""
    lines, expect = [], {}
    step = 0
    peak = 0

    def emit(entries, end, live_tokens):
        nonlocal step, peak
        peak = max(peak, live_tokens)
        lines.append(json.dumps({"step": step, "entries": [{"id": i, "tokens": t, "want": w} for i, t, w, _ in entries], "end": end}))
        exp = [(req, p) for _, _, w, (req, base) in entries for p in [base + x for x in w]]
        if exp:
            expect[step] = exp
        step += 1

    # 1. each request alone and whole
    for r, toks in enumerate(requests):
        emit([(f"whole{r}", toks, list(range(len(toks))), (r, 0))], [f"whole{r}"], round64(len(toks)))
    # 2. the last 32 tokens one by one
    for r, toks in enumerate(requests):
        n = len(toks)
        cut = max(1, n - 32)
        emit([(f"tail{r}", toks[:cut], list(range(cut)), (r, 0))], [], round64(n))
        for p in range(cut, n):
            emit([(f"tail{r}", [toks[p]], [0], (r, p))], [f"tail{r}"] if p == n - 1 else [], round64(n))
    # 3. batches of unequal lengths that start together; shorter requests end earlier; one batch after another
    order = list(range(len(requests)))
    for b, batch in enumerate((order[:3], order[3:])):
        prompt = {r: max(1, len(requests[r]) // 2 - r) for r in batch}
        live_tokens = sum(round64(len(requests[r])) for r in batch)
        emit([(f"b{b}r{r}", requests[r][:prompt[r]], list(range(prompt[r])), (r, 0)) for r in batch], [], live_tokens)
        pos = dict(prompt)
        live = list(batch)
        while live:
            entries = [(f"b{b}r{r}", [requests[r][pos[r]]], [0], (r, pos[r])) for r in live]
            for r in live:
                pos[r] += 1
            done = [r for r in live if pos[r] >= len(requests[r])]
            emit(entries, [f"b{b}r{r}" for r in done], sum(round64(len(requests[r])) for r in live))
            live = [r for r in live if r not in done]
    return lines, expect, peak


@pytest.mark.parametrize("name", ["tiny-a", "tiny-b"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_three_schedules(name, dtype, tmp_path):
    folder = model_folder(name, "bfloat16")
    plain = plain_model(folder)
    requests = [random_tokens(plain.V, n, 20 + i) for i, n in enumerate((40, 7, 95, 150, 33))]
    refs = [plain.forward(t) for t in requests]
    lines, expect, peak = build_trace(requests)
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                           "--max-tokens", str(peak)], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-3000:]
    done = [l for l in proc.stdout.splitlines() if l.startswith("done ")]
    assert done == [f"done {i}" for i in range(len(lines))]
    worst = 0.0
    for step in range(len(lines)):
        path = out / f"{step}.f32"
        if step not in expect:
            assert not path.exists()
            continue
        got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(len(expect[step]), plain.V).copy())
        ref = torch.stack([refs[r][p] for r, p in expect[step]])
        worst = max(worst, (got.double() - ref).abs().max().item())
    assert worst < TOL[dtype], worst


def test_replay_without_wanted_logits_writes_nothing(tmp_path):
    folder = model_folder("tiny-a", "bfloat16")
    lines = [json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3], "want": []}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "a", "tokens": [4], "want": [0]}], "end": ["a"]}),
             json.dumps({"step": 2, "entries": [], "end": []})]
    out = tmp_path / "o"
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", "64"], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert sorted(os.listdir(out)) == ["1.f32"] and os.path.getsize(out / "1.f32") == 256 * 4
    plain = plain_model(folder)
    got = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").copy())
    assert (got.double() - plain.forward([1, 2, 3, 4])[-1]).abs().max() < TOL["float32"]


def test_replay_bad_input_ends_with_one_line(tmp_path):
    folder = model_folder("tiny-a", "bfloat16")
    run = lambda text, model=folder: subprocess.run(
        [os.path.join(ROOT, "bin", "trace_run"), "--model", model, "--dtype", "float32", "--out", str(tmp_path / "o"),
         "--max-tokens", "64"], input=text, capture_output=True, text=True, timeout=300)
    ok = json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [1, 2], "want": [1]}], "end": []})
    cases = [("{not json\n", "input line 1"),
             (ok + "\n" + json.dumps({"step": 1, "entries": [{"id": "a", "tokens": [999], "want": [0]}], "end": []}) + "\n", "step 1.*vocabulary"),
             (ok + "\n" + json.dumps({"step": 1, "entries": [{"id": "a", "tokens": [3], "want": [4]}], "end": []}) + "\n", "step 1.*want"),
             (ok + "\n" + json.dumps({"step": 1, "entries": [{"id": "a", "want": [0]}], "end": []}) + "\n", "step 1.*tokens"),
             (json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [1] * 70, "want": []}], "end": []}) + "\n", "step 0.*full")]
    import re
    for text, pattern in cases:
        proc = run(text)
        lines = [l for l in proc.stderr.splitlines() if l.startswith("trace_run:")]
        assert proc.returncode == 1 and len(lines) == 1 and re.search(pattern, lines[0]), (pattern, proc.stderr[-500:])
        assert "Traceback" not in proc.stderr
    proc = run(ok + "\n", model=str(tmp_path / "nowhere"))
    assert proc.returncode == 1 and "cannot load" in proc.stderr and "Traceback" not in proc.stderr
