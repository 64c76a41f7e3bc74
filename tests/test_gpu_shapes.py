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
