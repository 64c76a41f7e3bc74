"""Gemma 2: typed configuration from config.json, and its plan.

What the reference's generic forward switches on for this architecture
(llama3.rs:13697-13703 embedding scale, 4634-4641 even layers slide,
5640-5642 score softcap, 14460-14465 and 14543-14548 post norms, 4530-4535
tanh-GELU gate, 14606-14611 logit softcap, 223-234 half-split rotation) is
written here once, as data for the builder.  Every number comes from
config.json; the defaults are the ones of the published Gemma 2 configs.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, asdict
from typing import Any, Mapping, Optional, Tuple

from .plan import (ConfigError, LayerPlan, ModelPlan, PartSpec, ScheduleEntry,
                   read_key, require)


@dataclass(frozen=True)
class Gemma2Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    max_position_embeddings: int = 8192
    rope_theta: float = 10000.0
    rms_norm_eps: float = 1e-6
    sliding_window: Optional[int] = 4096
    attn_logit_softcapping: Optional[float] = 50.0
    final_logit_softcapping: Optional[float] = 30.0
    query_pre_attn_scalar: float = 256.0
    hidden_activation: str = "gelu_pytorch_tanh"
    tie_word_embeddings: bool = True
    eos_token_id: Tuple[int, ...] = (1,)
    bos_token_id: Optional[int] = 2
    torch_dtype: str = "bfloat16"
    # Which layers slide, when config.json says so layer by layer ("sliding_attention" / "full_attention");
    # absent: even layers slide and odd layers see everything, the rule the reference has in code (llama3.rs:4634-4641).
    layer_types: Optional[Tuple[str, ...]] = None

    architecture = "Gemma2ForCausalLM"
    model_type = "gemma2"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Gemma2Config":
        V = read_key(d, "vocab_size", int)
        H = read_key(d, "hidden_size", int)
        L = read_key(d, "num_hidden_layers", int)
        nH = read_key(d, "num_attention_heads", int)
        nKV = read_key(d, "num_key_value_heads", int, nH)
        require(nH > 0, "num_attention_heads must be positive")
        hd = read_key(d, "head_dim", int, H // nH)
        I = read_key(d, "intermediate_size", int)
        # Keys that would change the arithmetic and that nothing here implements are refused, not dropped: the
        # projections have no biases (llama3.rs:14206-14217: the bias branches are no-ops for this architecture)
        # and the rotation has no scaling factors (no rope_freqs tensor, llama3.rs:5367-5378).
        require(not read_key(d, "attention_bias", bool, False),
                "attention_bias is true, and the attention projections here have no biases")
        require(d.get("rope_scaling") is None, f"rope_scaling {d.get('rope_scaling')!r} is not implemented (null only)")
        eos = d.get("eos_token_id", 1)
        if isinstance(eos, int) and not isinstance(eos, bool):
            eos = (eos,)
        elif isinstance(eos, (list, tuple)) and all(isinstance(e, int) for e in eos):
            eos = tuple(eos)
        elif eos is None:
            eos = ()
        else:
            raise ConfigError(f"config.json: key 'eos_token_id' must be an integer or a list of integers, found {eos!r}")
        kinds = d.get("layer_types")
        if kinds is not None:
            if not isinstance(kinds, (list, tuple)) or not all(isinstance(k, str) for k in kinds):
                raise ConfigError(f"config.json: key 'layer_types' must be a list of strings, found {kinds!r}")
            kinds = tuple(kinds)
        cfg = cls(
            vocab_size=V, hidden_size=H, num_hidden_layers=L, num_attention_heads=nH,
            num_key_value_heads=nKV, head_dim=hd, intermediate_size=I,
            max_position_embeddings=read_key(d, "max_position_embeddings", int, 8192),
            rope_theta=read_key(d, "rope_theta", float, 10000.0),
            rms_norm_eps=read_key(d, "rms_norm_eps", float, 1e-6),
            sliding_window=read_key(d, "sliding_window", int, 4096, allow_none=True),
            attn_logit_softcapping=read_key(d, "attn_logit_softcapping", float, 50.0, allow_none=True),
            final_logit_softcapping=read_key(d, "final_logit_softcapping", float, 30.0, allow_none=True),
            query_pre_attn_scalar=read_key(d, "query_pre_attn_scalar", float, float(hd)),
            hidden_activation=read_key(d, "hidden_activation", str,
                                       read_key(d, "hidden_act", str, "gelu_pytorch_tanh")),
            tie_word_embeddings=read_key(d, "tie_word_embeddings", bool, True),
            eos_token_id=eos,
            bos_token_id=read_key(d, "bos_token_id", int, 2, allow_none=True),
            torch_dtype=read_key(d, "torch_dtype", str, read_key(d, "dtype", str, "bfloat16")),
            layer_types=kinds,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for k in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                  "num_key_value_heads", "head_dim", "intermediate_size", "max_position_embeddings"):
            require(getattr(self, k) >= 1, f"{k} must be at least 1, found {getattr(self, k)}")
        require(self.num_attention_heads % self.num_key_value_heads == 0,
                f"num_key_value_heads ({self.num_key_value_heads}) must divide "
                f"num_attention_heads ({self.num_attention_heads})")
        require(self.head_dim % 2 == 0, f"head_dim must be even for the rotation, found {self.head_dim}")
        require(self.sliding_window is None or self.sliding_window >= 1,
                f"sliding_window must be at least 1 or null, found {self.sliding_window}")
        for k in ("attn_logit_softcapping", "final_logit_softcapping"):
            v = getattr(self, k)
            require(v is None or v > 0, f"{k} must be positive or null, found {v}")
        require(self.rms_norm_eps > 0, "rms_norm_eps must be positive")
        require(self.rope_theta > 0, "rope_theta must be positive")
        require(self.query_pre_attn_scalar > 0, "query_pre_attn_scalar must be positive")
        require(self.hidden_activation == "gelu_pytorch_tanh",
                f"hidden_activation must be 'gelu_pytorch_tanh' for Gemma 2, found '{self.hidden_activation}'")
        if self.layer_types is not None:
            require(len(self.layer_types) == self.num_hidden_layers,
                    f"layer_types names {len(self.layer_types)} layers, num_hidden_layers is {self.num_hidden_layers}")
            bad = sorted(set(self.layer_types) - {"sliding_attention", "full_attention"})
            require(not bad, f"layer_types holds {bad}: only 'sliding_attention' and 'full_attention' have a kernel")
        require(self.torch_dtype in ("bfloat16", "float32"),
                f"torch_dtype must be 'bfloat16' or 'float32', found '{self.torch_dtype}'")

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = [self.architecture]
        d["model_type"] = self.model_type
        d["eos_token_id"] = list(self.eos_token_id) if len(self.eos_token_id) != 1 else self.eos_token_id[0]
        if self.layer_types is None:
            del d["layer_types"]
        else:
            d["layer_types"] = list(self.layer_types)
        return d

    # ------------------------------------------------------------------ derived
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def layer_window(self, i: int) -> Optional[int]:
        """Even layers slide, odd layers are global (llama3.rs:4636-4641), unless layer_types says otherwise."""
        if self.layer_types is not None:
            return self.sliding_window if self.layer_types[i] == "sliding_attention" else None
        return self.sliding_window if i % 2 == 0 else None

    # ------------------------------------------------------------------ the plan
    def plan(self) -> ModelPlan:
        H = self.hidden_size
        norm = lambda name: PartSpec("rmsnorm", {"dim": H, "eps": self.rms_norm_eps,
                                                 "weight_offset": 1.0}, name)
        layers = []
        for i in range(self.num_hidden_layers):
            mixer = PartSpec("attention", {
                "hidden_size": H,
                "num_heads": self.num_attention_heads,
                "num_kv_heads": self.num_key_value_heads,
                "head_dim": self.head_dim,
                "scale": self.query_pre_attn_scalar ** -0.5,
                "softcap": self.attn_logit_softcapping,
                "window": self.layer_window(i),
                "position": "rope",
            }, "self_attn")
            ff = PartSpec("gated_mlp", {
                "hidden_size": H,
                "intermediate_size": self.intermediate_size,
                "activation": "gelu_tanh",
            }, "mlp")
            layers.append(LayerPlan(
                block="sandwich", mixer=mixer, feed_forward=ff,
                norms={"pre_mixer": norm("input_layernorm"),
                       "post_mixer": norm("post_attention_layernorm"),
                       "pre_ff": norm("pre_feedforward_layernorm"),
                       "post_ff": norm("post_feedforward_layernorm")},
                prefix=f"model.layers.{i}."))
        return ModelPlan(
            vocab_size=self.vocab_size,
            hidden_size=H,
            max_positions=self.max_position_embeddings,
            # sqrt taken of the width as an f32, as the reference does (llama3.rs:13697-13703)
            embedding=PartSpec("embedding", {"vocab_size": self.vocab_size, "dim": H,
                                             "scale": _f32(math.sqrt(H))}, "model.embed_tokens"),
            positions={"rope": PartSpec("rope", {"dim": self.head_dim, "theta": self.rope_theta,
                                                 "max_positions": self.max_position_embeddings})},
            layers=tuple(layers),
            schedule=tuple(ScheduleEntry(i) for i in range(self.num_hidden_layers)),
            final_norm=norm("model.norm"),
            head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "dim": H,
                                      "softcap": self.final_logit_softcapping,
                                      "tied_to": "model.embed_tokens" if self.tie_word_embeddings else None},
                          "lm_head"),
            stop_token_ids=tuple(self.eos_token_id),
        )


def _f32(x: float) -> float:
    import struct
    return struct.unpack("f", struct.pack("f", x))[0]
