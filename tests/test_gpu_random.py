"""Random configurations and schedules (seeded): sizes, options and batch shapes that nobody thought of, the
engine in both dtypes against the plain implementation.  Every case draws head size, heads and groups, widths,
vocabulary, number of layers, caps, window, eps and scale, then a batch of unequal prompts (sometimes in two
pieces), some decode steps, and runs it twice so that the second run finds used slots and pages."""
import os
import random
import tempfile

import pytest
import torch

import alice_llm_amd as alice
from helpers import TOL, max_err, plain_model, random_tokens

pytestmark = pytest.mark.gpu
_TMP = tempfile.TemporaryDirectory(prefix="alice_random_")


def draw(rng, big):
    d = rng.choice([64, 128, 256]) if big else rng.choice([16, 32, 48, 64, 80, 96, 128])
    nKV, group = rng.choice([1, 2, 3, 4]), rng.choice([1, 2, 3, 4])
    return dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", hidden_activation="gelu_pytorch_tanh",
                tie_word_embeddings=True, eos_token_id=1, bos_token_id=2, rope_theta=rng.choice([100.0, 10000.0]),
                attn_logit_softcapping=rng.choice([None, 5.0, 50.0]), final_logit_softcapping=rng.choice([None, 30.0]),
                rms_norm_eps=rng.choice([1e-6, 1e-5]), max_position_embeddings=512,
                num_hidden_layers=rng.choice([1, 2, 3]),
                hidden_size=rng.choice([256, 320, 512] if big else [24, 40, 64, 72, 96, 100, 128, 160, 256]),
                num_attention_heads=nKV * group, num_key_value_heads=nKV, head_dim=d,
                intermediate_size=rng.choice([512, 1024, 2048] if big else [17, 40, 64, 96, 136, 200, 256]),
                vocab_size=rng.choice([99, 257, 300, 512, 1001]),
                sliding_window=rng.choice([None, 3, 17, 64, 100]), query_pre_attn_scalar=rng.choice([d, 7, 144]))


@pytest.mark.parametrize("case", [f"small-{i}" for i in range(14)] + [f"big-{i}" for i in range(6)])
def test_random_configuration_and_schedule(case):
    big, number = case.startswith("big"), int(case.split("-")[1])
    rng = random.Random(case)
    raw = draw(rng, big)
    folder = os.path.join(_TMP.name, case)
    alice.write_random_model(folder, dict(raw), seed=number)
    plain = plain_model(folder)
    n_seq = rng.choice([1, 2, 3, 5])
    lens = [rng.choice([1, 17, 64, 65, 130, 200] if big else [1, 2, 15, 16, 17, 33, 64, 65, 100, 130]) for _ in range(n_seq)]
    decode = rng.choice([0, 1, 3, 20])
    cut = rng.choice([0, 0, 1, 7, 64, 70])
    seqs = [random_tokens(plain.V, n + decode, 100 * number + i) for i, n in enumerate(lens)]
    refs = [plain.forward(s) for s in seqs]
    scale = max(1.0, max(float(r.abs().max()) for r in refs))
    for dtype in ("float32", "bfloat16"):
        model = alice.load(folder, dtype=dtype)
        eng = model.engine(max_tokens=sum(-(-len(s) // 64) * 64 for s in seqs) + 64, max_seqs=n_seq + 1)
        for again in range(2):
            slots = eng.open(n_seq)
            if again:
                slots = slots[::-1]
            got = [[] for _ in seqs]
            pieces = [(0, cut), (cut, None)] if cut and all(n > cut for n in lens) else [(0, None)]      # a second piece on a cached prefix
            for a, b in pieces:
                ends = [n if b is None else b for n in lens]
                out, o = eng.step(slots, [s[a:e] for s, e in zip(seqs, ends)], "all"), 0
                for i, e in enumerate(ends):
                    got[i].append(out[o:o + e - a])
                    o += e - a
            for t in range(decode):
                out = eng.step(slots, [[s[n + t]] for s, n in zip(seqs, lens)], "last")
                for i in range(n_seq):
                    got[i].append(out[i:i + 1])
            eng.close(slots)
            for i in range(n_seq):
                err = max_err(torch.cat(got[i]), refs[i])
                assert err < TOL[dtype] * scale, (case, dtype, again, i, err, raw, lens, decode, cut)
        eng.cache.check_consistent()
        del eng, model
