"""Shared by the tests: two tiny Gemma 2 configurations that differ in every size and option, model
folders with random weights in a temporary place, and comparison helpers."""
import json
import os
import tempfile

import torch

_COMMON = dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", hidden_activation="gelu_pytorch_tanh",
               tie_word_embeddings=True, eos_token_id=1, bos_token_id=2)

# layers 2 / 3 (sliding, global / sliding, global, sliding), width 64 / 96, heads 4 / 6, kv heads 1 / 3
# (groups of 4 / 2), head size 16 / 24 (q width = width / != width), feed-forward 128 / 320, vocabulary
# 256 / 384, theta 1e4 / 5e5, window 8 / 6, score scale 16 (= head size) / 32 (!= head size),
# score cap 50 / 20, logit cap 30 / 15, eps 1e-6 / 1e-5.
TINY_A = dict(_COMMON, num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=1,
              head_dim=16, intermediate_size=128, vocab_size=256, rope_theta=10000.0, sliding_window=8,
              query_pre_attn_scalar=16, attn_logit_softcapping=50.0, final_logit_softcapping=30.0,
              rms_norm_eps=1e-6, max_position_embeddings=512)
TINY_B = dict(_COMMON, num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=3,
              head_dim=24, intermediate_size=320, vocab_size=384, rope_theta=500000.0, sliding_window=6,
              query_pre_attn_scalar=32, attn_logit_softcapping=20.0, final_logit_softcapping=15.0,
              rms_norm_eps=1e-5, max_position_embeddings=768)
# A third shape whose sizes suit the matrix-core kernels (head size 64, widths multiples of 32) but are
# no powers of two, with a window longer than a page.
TINY_C = dict(_COMMON, num_hidden_layers=4, hidden_size=160, num_attention_heads=6, num_key_value_heads=2,
              head_dim=64, intermediate_size=416, vocab_size=1000, rope_theta=20000.0, sliding_window=80,
              query_pre_attn_scalar=48, attn_logit_softcapping=12.0, final_logit_softcapping=9.0,
              rms_norm_eps=2e-6, max_position_embeddings=1024)
# The options that the published Gemma 2 configurations leave at their defaults, all turned the other way: a head with
# a matrix of its own, no caps, and the layers' kinds listed in config.json (global first, then two sliding layers).
TINY_D = dict(TINY_B, tie_word_embeddings=False, attn_logit_softcapping=None, final_logit_softcapping=None,
              layer_types=["full_attention", "sliding_attention", "sliding_attention"], sliding_window=5, hidden_size=80,
              num_attention_heads=4, num_key_value_heads=4, head_dim=32, query_pre_attn_scalar=32, vocab_size=130)
TINY = {"tiny-a": (TINY_A, 0), "tiny-b": (TINY_B, 1), "tiny-c": (TINY_C, 2), "tiny-d": (TINY_D, 3)}

_FOLDERS = {}
_TMP = None


def model_folder(name: str, stored: str = "bfloat16", hot: float = 1.0) -> str:
    """A folder with config.json and model.safetensors for a tiny configuration; made once per session.
    hot > 1 multiplies q/k and embedding weights so that scores and logits reach their caps."""
    global _TMP
    key = (name, stored, hot)
    if key in _FOLDERS:
        return _FOLDERS[key]
    import alice_llm_amd as alice
    if _TMP is None:
        _TMP = tempfile.TemporaryDirectory(prefix="alice_tests_")
    folder = os.path.join(_TMP.name, f"{name}-{stored}-{hot}")
    raw, seed = TINY[name]
    alice.write_random_model(folder, dict(raw), seed, {"bfloat16": torch.bfloat16, "float32": torch.float32}[stored])
    if hot != 1.0:
        from safetensors.torch import load_file, save_file
        path = os.path.join(folder, "model.safetensors")
        t = load_file(path)
        for k in t:
            if "q_proj" in k or "k_proj" in k or "embed_tokens" in k:
                t[k] = (t[k].float() * hot).to(t[k].dtype)
        save_file(t, path)
    _FOLDERS[key] = folder
    return folder


def write_marker_model(folder: str, raw: dict, seed: int, markers=(7, 8, 9)) -> None:
    """A model folder with random weights, edited so that the keys of the marker tokens stand out: every query scores
    them far above all other keys (one hidden feature that only the markers' embeddings have, read by one row of
    every key projection; a constant feature read by the matching row of every query projection; the pair sits in
    the rotation's slowest plane, so the score survives thousands of positions).  Among thousands of keys with nearly
    equal weights one key more or less changes nothing that a tolerance sees; one marker more or less does."""
    import alice_llm_amd as alice
    from safetensors.torch import load_file, save_file
    alice.write_random_model(folder, dict(raw), seed=seed)
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    d, nH, nKV = raw["head_dim"], raw["num_attention_heads"], raw["num_key_value_heads"]
    E = t["model.embed_tokens.weight"].float()
    E[:, 0] = 0.1                       # a feature every token has
    E[:, 1:2 + len(markers)] = 0.0
    for n, m in enumerate(markers):
        E[m, 1] = 0.5                   # one that only the markers have, which the keys read,
        E[m, 2 + n] = 0.5               # and one of its own for each marker, so that their values differ
    t["model.embed_tokens.weight"] = E.to(torch.bfloat16)
    j = d // 2 - 1                      # the slowest plane of the rotation: rows j and j + d/2 of a head
    for i in range(raw["num_hidden_layers"]):
        q = t[f"model.layers.{i}.self_attn.q_proj.weight"].float()
        k = t[f"model.layers.{i}.self_attn.k_proj.weight"].float()
        for h in range(nH):
            q[h * d + j, 0] += 2.0
        for h in range(nKV):
            k[h * d + j, 1] += 2.0
        t[f"model.layers.{i}.self_attn.q_proj.weight"] = q.to(torch.bfloat16)
        t[f"model.layers.{i}.self_attn.k_proj.weight"] = k.to(torch.bfloat16)
    save_file(t, path)


def plain_model(folder: str, dense: bool = False, device="cpu"):
    """dense: attention as one masked matrix product per head instead of key by key (the two forms are tested
    against each other); what sequences of thousands of tokens need."""
    from plain.gemma2_plain import PlainGemma2
    return PlainGemma2.from_folder(folder, dense=dense, device=device)


def random_tokens(vocab: int, n: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# Tolerances on logits, absolute, against the 64-bit plain implementation.
#   float32: sums of a few hundred 32-bit products and two dozen ops deep: errors stay near 1e-6 for
#            logits of order 1; 2e-5 leaves an order of magnitude.
#   bfloat16: activations are rounded to 8 bits of mantissa (relative 2^-9) between kernels; through a few
#            layers the logits (of order 1) carry errors of a few 1e-3 to 1e-2; a wrong mask, position or
#            head gives errors of order 0.1 to 1.
TOL = {"float32": 2e-5, "bfloat16": 3e-2}


def max_err(a: torch.Tensor, b: torch.Tensor) -> float:
    return (a.double().cpu() - b.double().cpu()).abs().max().item()


def model_from_tensors(cfg, tensors, dtype):
    """A model of the package filled with given tensors (by name, on the device), as the loader fills it from a folder."""
    from alice_llm_amd.api import Model
    from alice_llm_amd.engine.model import CausalLM
    from alice_llm_amd.parts import Precision
    lm = CausalLM(cfg.plan(), Precision.of(dtype), next(iter(tensors.values())).device)
    for name in lm.param_specs():
        lm.assign(name, tensors[name])
    lm.finalize()
    return Model(cfg, lm)
