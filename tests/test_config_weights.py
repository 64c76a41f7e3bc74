"""Configuration, registry, safetensors reading and the loader's errors (no GPU)."""
import json
import os
import struct

import pytest
import torch

import alice_llm_amd as alice
from alice_llm_amd.config import ConfigError, architecture_name
from alice_llm_amd.weights.loader import WeightError, check_tensors, random_tensors, _specs_without_device
from alice_llm_amd.weights.safetensors_io import SafetensorsFile, TensorSource, WeightFileError, write_safetensors
from helpers import TINY_A, TINY_B, model_folder


def test_presets_parse_and_derive():
    for name in alice.preset_names():
        cfg = alice.config_from_dict(alice.preset(name))
        plan = cfg.plan()
        assert len(plan.layers) == cfg.num_hidden_layers == len(plan.schedule)
        assert [l.mixer.args["window"] for l in plan.layers[:3]] == [cfg.sliding_window, None, cfg.sliding_window][:len(plan.layers[:3])]
    c = alice.config_from_dict(alice.preset("27b"))
    assert c.q_dim == 4096 and c.kv_dim == 2048 and abs(c.plan().layers[0].mixer.args["scale"] - 144 ** -0.5) < 1e-12
    b = alice.config_from_dict(dict(TINY_B)).plan()
    assert b.layers[0].mixer.args["scale"] == 32 ** -0.5 and b.layers[1].mixer.args["window"] is None
    assert b.embedding.args["scale"] == float(torch.tensor(96.0).sqrt())            # sqrt taken in f32
    assert b.head.args["softcap"] == 15.0 and b.head.args["tied_to"] == "model.embed_tokens"
    assert b.layers[2].norms["post_ff"].args == {"dim": 96, "eps": 1e-5, "weight_offset": 1.0}


def test_config_defaults_and_nulls():
    d = {k: v for k, v in TINY_A.items() if k not in ("head_dim", "num_key_value_heads", "rope_theta", "rms_norm_eps",
                                                       "sliding_window", "query_pre_attn_scalar", "attn_logit_softcapping")}
    c = alice.config_from_dict(dict(d, unknown_key=123))
    assert c.head_dim == 16 and c.num_key_value_heads == 4 and c.rope_theta == 10000.0 and c.rms_norm_eps == 1e-6
    assert c.sliding_window == 4096 and c.query_pre_attn_scalar == 16.0 and c.attn_logit_softcapping == 50.0
    c = alice.config_from_dict(dict(TINY_A, sliding_window=None, attn_logit_softcapping=None, eos_token_id=[1, 107]))
    assert c.sliding_window is None and c.attn_logit_softcapping is None and c.eos_token_id == (1, 107)
    assert all(l.mixer.args["window"] is None for l in c.plan().layers) and c.plan().stop_token_ids == (1, 107)
    assert alice.config_from_dict(c.to_dict()) == c


@pytest.mark.parametrize("change, word", [
    ({"hidden_size": None}, "hidden_size"), ({"vocab_size": "256"}, "vocab_size"),
    ({"num_key_value_heads": 3}, "divide"), ({"head_dim": 15}, "even"), ({"sliding_window": 0}, "sliding_window"),
    ({"final_logit_softcapping": -1.0}, "final_logit_softcapping"), ({"hidden_activation": "silu"}, "gelu_pytorch_tanh"),
    ({"architectures": ["LlamaForCausalLM"]}, "registered"), ({"num_hidden_layers": True}, "integer"),
    # keys that would change the arithmetic and that nothing implements are refused, not dropped
    ({"layer_types": ["sliding_attention"]}, "layer_types names 1"), ({"layer_types": ["full_attention", "chunked"]}, "chunked"),
    ({"attention_bias": True}, "attention_bias"), ({"rope_scaling": {"type": "linear", "factor": 2.0}}, "rope_scaling"),
])
def test_config_errors_name_the_key(change, word):
    d = dict(TINY_A)
    for k, v in change.items():
        if v is None:
            d.pop(k)
        else:
            d[k] = v
    with pytest.raises(ConfigError, match=word):
        alice.config_from_dict(d)


def test_layer_kinds_from_config_when_it_lists_them():
    c = alice.config_from_dict(dict(TINY_B, layer_types=["full_attention", "sliding_attention", "sliding_attention"], dtype="float32"))
    assert [l.mixer.args["window"] for l in c.plan().layers] == [None, 6, 6] and c.torch_dtype == "float32"
    assert alice.config_from_dict(c.to_dict()) == c and "layer_types" not in alice.config_from_dict(dict(TINY_B)).to_dict()


def test_registry(tmp_path):
    assert "Gemma2ForCausalLM" in alice.registered_architectures()
    assert architecture_name({"model_type": "gemma2"}) == "Gemma2ForCausalLM"
    with pytest.raises(ConfigError, match="Gemma2ForCausalLM"):
        architecture_name({"model_type": "mystery"})
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        alice.load_config(str(tmp_path))


def test_safetensors_round_trip_against_the_library(tmp_path):
    from safetensors.torch import load_file, save_file
    ts = {"a": torch.randn(3, 5).bfloat16(), "b": torch.arange(7, dtype=torch.int32), "c": torch.randn(2, 2), "e": torch.zeros(0, 4)}
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, [(k, v.dtype, v.shape) for k, v in ts.items()], lambda k: ts[k])
    lib = load_file(path)
    assert all(torch.equal(lib[k], ts[k]) for k in ts)
    save_file(ts, str(tmp_path / "lib.safetensors"))
    f = SafetensorsFile(str(tmp_path / "lib.safetensors"))
    assert sorted(f.keys()) == sorted(ts) and all(torch.equal(f.tensor(k), ts[k]) for k in ts)
    assert f.info("a") == (torch.bfloat16, (3, 5))


def test_safetensors_errors(tmp_path):
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"abc")
    with pytest.raises(WeightFileError, match="truncated"):
        SafetensorsFile(str(p))
    p.write_bytes(struct.pack("<Q", 5) + b"{nope")
    with pytest.raises(WeightFileError, match="not JSON"):
        SafetensorsFile(str(p))
    hdr = json.dumps({"x": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(WeightFileError, match="truncated.*'x'"):
        SafetensorsFile(str(p))
    hdr = json.dumps({"x": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 4)
    with pytest.raises(WeightFileError, match="unknown dtype"):
        SafetensorsFile(str(p))
    with pytest.raises(WeightFileError, match="neither"):
        TensorSource(str(tmp_path / "nowhere"))


def test_weight_error_lists_everything_at_once():
    specs = _specs_without_device(alice.config_from_dict(dict(TINY_A)))
    assert list(specs)[0] == "model.embed_tokens.weight" and "lm_head.weight" not in specs and len(specs) == 1 + 2 * 11 + 1
    found = {n: (torch.bfloat16, s.shape) for n, s in specs.items()}
    del found["model.layers.1.mlp.up_proj.weight"], found["model.norm.weight"]
    found["model.layers.0.self_attn.q_proj.weight"] = (torch.bfloat16, (64, 63))
    found["model.layers.0.self_attn.k_proj.weight"] = (torch.float16, (16, 64))
    found["model.layers.7.extra.weight"] = (torch.float32, (1,))
    with pytest.raises(WeightError) as e:
        check_tensors("folder", specs, found)
    msg = str(e.value)
    assert e.value.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.value.unexpected == ["model.layers.7.extra.weight"] and len(e.value.wrong) == 2
    for word in ("up_proj", "model.norm.weight", "extra", "[64, 63]", "float16", "expected shape [64, 64]"):
        assert word in msg
    untied = _specs_without_device(alice.config_from_dict(dict(TINY_A, tie_word_embeddings=False)))
    assert untied["lm_head.weight"].shape == (256, 64)
    # not strict: tensors that the model does not declare are handed back instead of refused, alone ...
    ok = {n: (torch.bfloat16, s.shape) for n, s in specs.items()}
    ok["rotary.inv_freq"] = (torch.float32, (8,))
    assert check_tensors("folder", specs, ok, strict=False) == ["rotary.inv_freq"]
    with pytest.raises(WeightError, match="unexpected \\(1\\): rotary.inv_freq"):
        check_tensors("folder", specs, ok)
    # ... and still listed beside any other problem
    del ok["model.norm.weight"]
    with pytest.raises(WeightError) as e:
        check_tensors("folder", specs, ok, strict=False)
    assert e.value.unexpected == ["rotary.inv_freq"] and e.value.missing == ["model.norm.weight"]


def test_a_head_size_beyond_the_kernels_is_refused_when_the_model_is_put_together():
    from alice_llm_amd.config import ConfigError
    cfg = alice.config_from_dict(dict(TINY_A, head_dim=272, query_pre_attn_scalar=272))
    with pytest.raises(ValueError, match="head_dim 272"):
        _specs_without_device(cfg)
    assert alice.config_from_dict(dict(TINY_A, attention_bias=False, rope_scaling=None)).head_dim == 16


def test_random_weights_folder():
    folder = model_folder("tiny-b", "bfloat16")
    again = model_folder("tiny-b", "float32")
    src, src32 = TensorSource(folder), TensorSource(again)
    cfg = alice.load_config(folder)
    assert cfg.torch_dtype == "bfloat16" and alice.load_config(again).torch_dtype == "float32"
    specs = _specs_without_device(cfg)
    assert sorted(src.keys()) == sorted(specs)
    e, n = src.tensor("model.embed_tokens.weight"), src.tensor("model.layers.2.input_layernorm.weight")
    assert e.dtype == torch.bfloat16 and src32.tensor("model.norm.weight").dtype == torch.float32
    assert abs(e.float().std().item() - 0.02) < 1e-3 and abs(n.float().std().item() - 0.1) < 0.03
    assert torch.equal(src32.tensor("model.embed_tokens.weight").bfloat16(), e)       # one stream, cast at the end
    a = dict(random_tensors(specs, 1, torch.float32))
    assert torch.equal(a["model.embed_tokens.weight"], src32.tensor("model.embed_tokens.weight"))
    b = dict(random_tensors(specs, 2, torch.float32))
    assert not torch.equal(a["model.norm.weight"], b["model.norm.weight"])


def test_sharded_folder(tmp_path):
    from safetensors.torch import save_file
    a = {"x.weight": torch.randn(4, 3).bfloat16()}
    b = {"y.weight": torch.randn(5)}
    save_file(a, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file(b, str(tmp_path / "model-00002-of-00002.safetensors"))
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {
        "x.weight": "model-00001-of-00002.safetensors", "y.weight": "model-00002-of-00002.safetensors"}}))
    src = TensorSource(str(tmp_path))
    assert sorted(src.keys()) == ["x.weight", "y.weight"] and torch.equal(src.tensor("y.weight"), b["y.weight"])
    assert src.info("x.weight") == (torch.bfloat16, (4, 3))
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"x.weight": "missing.safetensors"}}))
    with pytest.raises(WeightFileError, match="missing.safetensors"):
        TensorSource(str(tmp_path))


def test_a_library_from_other_sources_is_not_used(tmp_path, monkeypatch):
    """The library carries a digest of its sources and flags: the bindings use a built library only if the
    digest is that of the sources beside them (a library left from an edit or an older checkout is not)."""
    from alice_llm_amd.csrc import build
    from alice_llm_amd.hip import ops
    d0 = build.source_digest()
    assert len(d0) == 32 and d0 == build.source_digest()
    src = tmp_path / "csrc"
    src.mkdir()
    (src / "a.hip").write_text("int x;")
    (src / "a.h").write_text("")
    monkeypatch.setattr(build, "HERE", str(src))
    d1 = build.source_digest()
    (src / "a.h").write_text("// edited")
    d2 = build.source_digest()
    monkeypatch.setattr(build, "FLAGS", build.FLAGS + ["-O0"])
    assert len({d0, d1, d2, build.source_digest()}) == 4

    class Old:                                    # a library from before the digest existed
        pass

    class Built:
        def __init__(self, d):
            self.alice_source_digest = lambda: d.encode()
    assert not ops._built_from_these_sources(Old())
    assert not ops._built_from_these_sources(Built(d2))
    assert ops._built_from_these_sources(Built(build.source_digest()))
