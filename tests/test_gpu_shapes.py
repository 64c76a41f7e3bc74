"""The real models' layer widths (Gemma 2 2B, 9B and 27B: head sizes 256 and 128, widths 2304 / 3584 /
4608 that are no powers of two, query width != width, score scale != head size for 27B) with few layers
and a small vocabulary, against the plain implementation, whole and token by token, in both dtypes."""
import os
import tempfile

import pytest
import torch

import alice_llm_amd as alice
from helpers import TOL, max_err, plain_model, random_tokens

pytestmark = pytest.mark.gpu

_COMMON = dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", hidden_activation="gelu_pytorch_tanh",
               tie_word_embeddings=True, eos_token_id=1, bos_token_id=2, rope_theta=10000.0,
               attn_logit_softcapping=50.0, final_logit_softcapping=30.0, rms_norm_eps=1e-6, max_position_embeddings=512)
WIDE = {
    "2b-wide": dict(_COMMON, num_hidden_layers=2, hidden_size=2304, num_attention_heads=8, num_key_value_heads=4,
                    head_dim=256, intermediate_size=9216, vocab_size=4000, sliding_window=70, query_pre_attn_scalar=256),
    "9b-wide": dict(_COMMON, num_hidden_layers=2, hidden_size=3584, num_attention_heads=16, num_key_value_heads=8,
                    head_dim=256, intermediate_size=14336, vocab_size=2000, sliding_window=90, query_pre_attn_scalar=256),
    "27b-wide": dict(_COMMON, num_hidden_layers=1, hidden_size=4608, num_attention_heads=32, num_key_value_heads=16,
                     head_dim=128, intermediate_size=36864, vocab_size=2000, sliding_window=50, query_pre_attn_scalar=144),
}
_TMP = tempfile.TemporaryDirectory(prefix="alice_wide_")


@pytest.mark.parametrize("name", list(WIDE))
def test_real_widths_whole_and_token_by_token(name):
    folder = os.path.join(_TMP.name, name)
    alice.write_random_model(folder, dict(WIDE[name]), seed=3)
    plain = plain_model(folder)
    toks = random_tokens(plain.V, 110, 60)
    ref = plain.forward(toks)
    scale = max(1.0, float(ref.abs().max()))
    for dtype in ("float32", "bfloat16"):
        model = alice.load(folder, dtype=dtype)
        eng = model.engine(max_tokens=256, max_seqs=2)
        s = eng.open(1)
        whole = eng.step(s, [toks], "all")
        eng.close(s)
        s = eng.open(2)                              # a second, shorter sequence shares the batch
        cut = [eng.step(s, [toks[:100], toks[5:40]], [list(range(100)), []])]
        for t in toks[100:]:
            cut.append(eng.step(s, [[t], [7]], [[0], []]))
        eng.close(s)
        cut = torch.cat(cut)
        assert max_err(whole, ref) < TOL[dtype] * scale, (dtype, max_err(whole, ref))
        assert max_err(cut, ref) < TOL[dtype] * scale, (dtype, max_err(cut, ref))
        del model, eng
        torch.cuda.empty_cache()


ODD = {
    # a width that is no multiple of 8, as many groups as heads, a vocabulary of 257
    "width-100": dict(_COMMON, num_hidden_layers=2, hidden_size=100, num_attention_heads=5, num_key_value_heads=5, head_dim=16,
                      intermediate_size=136, vocab_size=257, sliding_window=9, query_pre_attn_scalar=16),
    # a head size that is a multiple of 16 and not of 32, three heads on one group
    "head-80": dict(_COMMON, num_hidden_layers=2, hidden_size=160, num_attention_heads=6, num_key_value_heads=2, head_dim=80,
                    intermediate_size=200, vocab_size=300, sliding_window=33, query_pre_attn_scalar=80),
    # query width three times the width, an odd feed-forward width, a scale that is not the head size
    "head-96": dict(_COMMON, num_hidden_layers=1, hidden_size=64, num_attention_heads=2, num_key_value_heads=2, head_dim=96,
                    intermediate_size=17, vocab_size=99, sliding_window=5, query_pre_attn_scalar=7),
    # forty heads into a width of 24: the output projection's inner dimension is a hundred times its outputs
    "heads-40": dict(_COMMON, num_hidden_layers=2, hidden_size=24, num_attention_heads=40, num_key_value_heads=5, head_dim=64,
                     intermediate_size=40, vocab_size=130, sliding_window=50, query_pre_attn_scalar=64),
}


@pytest.mark.parametrize("name", list(ODD))
def test_odd_sizes_whole_and_token_by_token(name):
    """Sizes that fit no tile: every kernel takes them (or hands over to one that does); none gives a wrong result."""
    folder = os.path.join(_TMP.name, name)
    alice.write_random_model(folder, dict(ODD[name]), seed=4)
    plain = plain_model(folder)
    toks = random_tokens(plain.V, 90, 61)
    ref = plain.forward(toks)
    scale = max(1.0, float(ref.abs().max()))
    for dtype in ("float32", "bfloat16"):
        model = alice.load(folder, dtype=dtype)
        eng = model.engine(max_tokens=256, max_seqs=2)
        s = eng.open(1)
        whole = eng.step(s, [toks], "all")
        eng.close(s)
        s = eng.open(1)
        cut = [eng.step(s, [toks[:70]], "all")] + [eng.step(s, [[t]], "last") for t in toks[70:]]
        eng.close(s)
        assert max_err(whole, ref) < TOL[dtype] * scale, (dtype, max_err(whole, ref))
        assert max_err(torch.cat(cut), ref) < TOL[dtype] * scale, (dtype, max_err(torch.cat(cut), ref))


def test_full_2b_shape_bfloat16_against_the_32_bit_path():
    """The whole Gemma 2 2B shape (26 layers, vocabulary 256,000) with random weights: a prompt of 292 tokens and
    8 single tokens, the bfloat16 path against the true 32-bit path on the same weights.  The reference checks its
    quantised forward against an all-f32 one the same way (examples/test_1b.rs:190-227: max and mean difference
    of the logits).  Bound: the logits (rms about 1, maximum about 8) differ by at most 0.06, and where the
    two paths choose another token the 32-bit logits of the two are closer than that."""
    free, _ = torch.cuda.mem_get_info()
    if free < 40e9:
        pytest.skip(f"needs 40 GB of free GPU memory for both models, {free / 1e9:.0f} GB are free")
    cfg = alice.config_from_dict(alice.preset("2b"))
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.vocab_size, cfg.head_dim) == (26, 2304, 256000, 256)
    toks = random_tokens(cfg.vocab_size, 300, 62)
    outs = {}
    for dtype in ("float32", "bfloat16"):
        model = alice.Model.random(cfg, seed=0, dtype=dtype, fast=True)       # the same bfloat16 weights for both paths
        eng = model.engine(seq_lens=[320], max_seqs=1)
        s = eng.open(1)
        got = [eng.step(s, [toks[:292]], "all")] + [eng.step(s, [[t]], "last").clone() for t in toks[292:]]
        outs[dtype] = torch.cat(got).cpu()
        del eng, model
        torch.cuda.empty_cache()
    f, b = outs["float32"], outs["bfloat16"]
    assert f.shape == (300, 256000) and 0.5 < float(f.pow(2).mean().sqrt()) < 2.0 and float(f.abs().max()) > 4.0
    diff = (f - b).abs()
    assert float(diff.max()) <= 0.06, float(diff.max())
    assert float(diff.pow(2).mean().sqrt()) < 0.012
    fa, ba = f.argmax(-1), b.argmax(-1)
    for p in (fa != ba).nonzero().flatten().tolist():
        assert float(f[p, fa[p]] - f[p, ba[p]]) < 0.06, p
    assert int((fa != ba).sum()) <= 3
