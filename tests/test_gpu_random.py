"""Random configurations and schedules (seeded): sizes, options and batch shapes that nobody thought of, the
engine in both dtypes against the plain implementation.  Every case draws head size, heads and groups, widths,
vocabulary, number of layers, caps, window, eps and scale, then a batch of unequal prompts (sometimes in two
pieces), some decode steps, and runs it twice so that the second run finds used slots and pages.  A second set of
cases has the widths of real models and batches of up to 70 sequences: the 32-bit path against the plain
implementation, and bfloat16 against the 32-bit path."""
import os
import random
import tempfile

import pytest
import torch

import alice_llm_amd as alice
from helpers import TOL, max_err, model_from_tensors, plain_model, random_tokens

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


@pytest.mark.parametrize("case", [f"wide-{i}" for i in range(8)])
def test_random_widths_of_real_models_in_batches_up_to_70(case):
    """Widths, head counts and feed-forward widths as real models have them (one or two layers, a small vocabulary),
    batches of 1 to 70 unequal prompts in one or two pieces, then single tokens through captured steps or eagerly,
    their ids from the host or on the device: this is where the rules that pick kernels and tiles by size take their
    branches.  Two comparisons.  The 32-bit path, every sequence alone and whole, against the plain implementation
    (float64 on the GPU, the same tensors) on up to 20 of the sequences; and the bfloat16 path in the batch against
    that 32-bit path on all of them: for the sequences past the twentieth the engine is its own reference, which a
    mistake common to both paths would pass (they are covered by the first twenty, which take the same code with
    other lengths).  The largest bfloat16 error stays below 8 % of the logits' rms (4 to 5.5 % over 900 such cases);
    a k-tile or a head left out is far above that."""
    number = int(case.split("-")[1])
    rng = random.Random(case)
    d = rng.choice([64, 128, 256])
    nKV, group = rng.choice([1, 2, 4, 8, 16]), rng.choice([1, 2, 4, 8])
    while nKV * group * d > 8192:
        if group > 1:
            group //= 2
        else:
            nKV //= 2
    V = rng.choice([1000, 2049, 4000])
    raw = dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", hidden_activation="gelu_pytorch_tanh",
               tie_word_embeddings=True, eos_token_id=1, bos_token_id=2, rope_theta=10000.0,
               attn_logit_softcapping=rng.choice([None, 50.0]), final_logit_softcapping=rng.choice([None, 30.0]),
               rms_norm_eps=1e-6, max_position_embeddings=1024, num_hidden_layers=rng.choice([1, 2]),
               hidden_size=rng.choice([1024, 1536, 2048, 2304, 3072, 3584, 4096, 4608]),
               num_attention_heads=nKV * group, num_key_value_heads=nKV, head_dim=d,
               intermediate_size=rng.choice([2048, 4096, 8192, 9216, 14336]), vocab_size=V,
               sliding_window=rng.choice([None, 64, 100, 300]), query_pre_attn_scalar=d)
    cfg = alice.config_from_dict(raw)
    n_seq = rng.choice([1, 8, 9, 16, 17, 33, 48, 64, 65, 70])
    lens = [rng.randint(1, rng.choice([20, 150, 400])) for _ in range(n_seq)]
    decode = rng.choice([1, 3, 12])
    seqs = [random_tokens(V, n + decode, 100 * number + i) for i, n in enumerate(lens)]
    from alice_llm_amd.engine.model import CausalLM
    from alice_llm_amd.weights.loader import random_tensors
    from plain.gemma2_plain import PlainGemma2
    dev = torch.device("cuda", torch.cuda.current_device())
    tensors = dict(random_tensors(CausalLM(cfg.plan(), "float32", "cpu").param_specs(), number, torch.bfloat16, dev))
    exact = model_from_tensors(cfg, tensors, "float32")
    eng = exact.engine(max_tokens=1024, max_seqs=1, use_graphs=False)
    refs = []
    for s in seqs:
        slot = eng.open(1)
        refs.append(eng.step(slot, [s], "all").cpu())
        eng.close(slot)
    del eng, exact
    plain = PlainGemma2(raw, tensors, dense=True, device=dev)
    for s, r in list(zip(seqs, refs))[:20]:
        want = plain.forward(s).float().cpu()
        assert max_err(r, want) < TOL["float32"] * max(1.0, float(want.abs().max())), (raw, len(s), max_err(r, want))
    del plain
    torch.cuda.empty_cache()
    rms = min(float(r.pow(2).mean().sqrt()) for r in refs)
    model = model_from_tensors(cfg, tensors, "bfloat16")
    eng = model.engine(seq_lens=[len(s) for s in seqs], max_seqs=n_seq, use_graphs=rng.random() < 0.7)
    for again in range(2):
        slots = eng.open(n_seq)
        rng.shuffle(slots)
        cut = [rng.randint(1, n) if again else n for n in lens]
        errs = []
        out = eng.step(slots, [s[:c] for s, c in zip(seqs, cut)], "last")
        errs += [max_err(out[i], refs[i][cut[i] - 1]) for i in range(n_seq)]
        rest = [i for i in range(n_seq) if cut[i] < lens[i]]
        if rest:
            out = eng.step([slots[i] for i in rest], [seqs[i][cut[i]:lens[i]] for i in rest], "last")
            errs += [max_err(out[j], refs[i][lens[i] - 1]) for j, i in enumerate(rest)]
        on_device = rng.random() < 0.5
        for k in range(decode):
            ids = [seqs[i][lens[i] + k] for i in range(n_seq)]
            feed = torch.tensor(ids, dtype=torch.int32, device=eng.device) if on_device else [[t] for t in ids]
            out = eng.step(slots, feed, "last")
            errs += [max_err(out[i], refs[i][lens[i] + k]) for i in range(n_seq)]
        eng.close(slots)
        eng.cache.check_consistent()
        assert max(errs) < 0.08 * rms, (raw, n_seq, lens, cut, max(errs), rms)
    del eng, model
    torch.cuda.empty_cache()
