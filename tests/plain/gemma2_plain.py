"""Plain, slow Gemma 2 for whole sequences: the oracle of the tests.

One function per formula, each written from the formula that the reference's
single-token CPU forward computes (its file:line in each docstring).  Whole
sequences, dense masks, no cache, float64 by default, and no code shared with
the package under test: it reads config.json keys and safetensors tensor names
itself.  It runs where its tensors are: on the CPU, or with `device` on a GPU
(torch's float64 there), which is what a model of full size needs.

Two deliberate differences from the reference's text, both part of this
architecture's contract rather than of the reference's GGUF convention:
  * RMSNorm multiplies by (1 + w): safetensors files hold w, while the GGUF
    files that the reference reads hold 1 + w already (llama3.rs:5244-5256
    multiplies by the stored value).
  * the attention scale is query_pre_attn_scalar ** -0.5; the reference
    hard-codes head_dim ** -0.5 (llama3.rs:5446), the same number whenever
    query_pre_attn_scalar == head_dim.
"""
from __future__ import annotations

import json
import math
import os

import torch

DT = torch.float64


# --------------------------------------------------------------------------- parts

def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * (1 + w), over the last axis.

    llama3.rs:5244-5256 (sum of squares, mean, 1/sqrt(mean+eps), multiply by the
    weight); the weight convention is (1 + w), see the module docstring.
    """
    ms = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * (1.0 / torch.sqrt(ms + eps)) * (1.0 + w)


def rope_half_split(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """Rotate pairs (j, j + d/2) of the last axis by positions * theta^(-2j/d).

    x: [T, heads, d]; positions: [T].  llama3.rs:5367-5378 (apply_rope_neox):
    freq_j = 1/theta^(2j/d); y[j] = x[j] cos - x[j+d/2] sin;
    y[j+d/2] = x[j] sin + x[j+d/2] cos.  Same pairing in src/rope.rs:12-27.
    """
    d = x.shape[-1]
    half = d // 2
    out = torch.empty_like(x)
    for j in range(half):
        freq = 1.0 / (theta ** (2.0 * j / d))
        ang = positions.to(x.dtype) * freq                      # [T]
        c = torch.cos(ang)[:, None]
        s = torch.sin(ang)[:, None]
        x0 = x[..., j]
        x1 = x[..., j + half]
        out[..., j] = x0 * c - x1 * s
        out[..., j + half] = x0 * s + x1 * c
    return out


def softcap(x: torch.Tensor, cap) -> torch.Tensor:
    """cap * tanh(x / cap); identity when cap is None.

    llama3.rs:5640-5642 (attention scores), llama3.rs:14606-14611 (final logits).
    """
    if cap is None:
        return x
    return cap * torch.tanh(x / cap)


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))).  llama3.rs:6183-6186."""
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x * x * x)))


def attention_core(q, k, v, scale, cap, window):
    """Causal grouped-query attention over one whole sequence, key by key.

    q: [T, nH, d]; k, v: [T, nKV, d], already rotated.  For the query at
    position p and head h: kv head h // (nH // nKV); keys t from
    max(0, p + 1 - window) to p inclusive (window None: from 0), so a window
    of W holds W keys, the query's own included (llama3.rs:5444-5451);
    score = (q . k_t) * scale, then softcap, then softmax over these keys,
    then the weighted sum of v_t (llama3.rs:5622-5688).
    """
    T, nH, d = q.shape
    nKV = k.shape[1]
    g = nH // nKV
    out = torch.zeros(T, nH, d, dtype=q.dtype, device=q.device)
    for p in range(T):
        start = 0 if window is None else max(0, p + 1 - window)
        for h in range(nH):
            kv = h // g
            s = (k[start:p + 1, kv, :] @ q[p, h, :]) * scale     # [n]
            s = softcap(s, cap)
            m = s.max()
            e = torch.exp(s - m)
            pr = e / e.sum()
            out[p, h, :] = pr @ v[start:p + 1, kv, :]
    return out


def attention_dense(q, k, v, scale, cap, window):
    """The same attention through one masked matrix product per head (second form; the one long sequences use)."""
    T, nH, d = q.shape
    nKV = k.shape[1]
    g = nH // nKV
    i = torch.arange(T, device=q.device)[:, None]
    j = torch.arange(T, device=q.device)[None, :]
    allowed = j <= i
    if window is not None:
        allowed = allowed & (j >= i + 1 - window)
    out = torch.empty(T, nH, d, dtype=q.dtype, device=q.device)
    for h in range(nH):
        s = (q[:, h, :] @ k[:, h // g, :].T) * scale
        s = softcap(s, cap)
        s = s.masked_fill(~allowed, float("-inf"))
        out[:, h, :] = torch.softmax(s, dim=-1) @ v[:, h // g, :]
    return out


def geglu(x, w_gate, w_up, w_down):
    """down( gelu_tanh(gate x) * (up x) ).  llama3.rs:14519-14540; activation on the gate branch."""
    return (gelu_tanh(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


# --------------------------------------------------------------------------- model

class PlainGemma2:
    """Whole-sequence forward from a model folder's raw config.json and tensors."""

    def __init__(self, config: dict, tensors: dict, dtype=DT, dense: bool = False, device="cpu"):
        c = config
        self.dtype = dtype
        self.device = torch.device(device)
        self.attention = attention_dense if dense else attention_core
        self.V = c["vocab_size"]
        self.H = c["hidden_size"]
        self.L = c["num_hidden_layers"]
        self.nH = c["num_attention_heads"]
        self.nKV = c.get("num_key_value_heads", self.nH)
        self.d = c.get("head_dim", self.H // self.nH)
        self.I = c["intermediate_size"]
        self.theta = float(c.get("rope_theta", 10000.0))
        self.eps = float(c.get("rms_norm_eps", 1e-6))
        self.window = c.get("sliding_window", 4096)
        self.cap_a = c.get("attn_logit_softcapping", 50.0)
        self.cap_f = c.get("final_logit_softcapping", 30.0)
        self.scale = float(c.get("query_pre_attn_scalar", self.d)) ** -0.5
        self.layer_types = c.get("layer_types")
        self.t = {k: v.to(device=self.device, dtype=dtype) for k, v in tensors.items()}

    @classmethod
    def from_folder(cls, folder: str, dtype=DT, dense: bool = False, device="cpu"):
        from safetensors import safe_open
        with open(os.path.join(folder, "config.json")) as f:
            config = json.load(f)
        tensors = {}
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
            for k in f.keys():
                tensors[k] = f.get_tensor(k)
        return cls(config, tensors, dtype, dense, device)

    def layer_window(self, i: int):
        """Even layers slide, odd layers see everything (llama3.rs:4634-4641); a config.json that lists
        layer_types layer by layer overrides the rule."""
        if self.layer_types is not None:
            return self.window if self.layer_types[i] == "sliding_attention" else None
        return self.window if i % 2 == 0 else None

    def embed(self, tokens):
        """Row copy times sqrt(hidden) taken in f32.  llama3.rs:13686-13703."""
        E = self.t["model.embed_tokens.weight"]
        scale = float(torch.tensor(float(self.H), dtype=torch.float32).sqrt())
        return E[torch.as_tensor(tokens, dtype=torch.long, device=self.device)] * scale

    def layer(self, i: int, x: torch.Tensor, positions: torch.Tensor, taps=None):
        """x + N_post_attn(Attn(N_in(x))), then x + N_post_ffn(FFN(N_pre_ffn(x))).

        llama3.rs:14178 (input norm), 14206-14217 (q, k, v), 14307-14328 (rope),
        14362-14378 (attention), 14423 (output projection), 14460-14470 (post
        norm, residual), 14497 (pre-ffn norm), 14519-14557 (GeGLU, post norm,
        residual).
        """
        t = self.t
        p = f"model.layers.{i}."
        T = x.shape[0]
        n = rms_norm(x, t[p + "input_layernorm.weight"], self.eps)
        q = (n @ t[p + "self_attn.q_proj.weight"].T).view(T, self.nH, self.d)
        k = (n @ t[p + "self_attn.k_proj.weight"].T).view(T, self.nKV, self.d)
        v = (n @ t[p + "self_attn.v_proj.weight"].T).view(T, self.nKV, self.d)
        q = rope_half_split(q, positions, self.theta)
        k = rope_half_split(k, positions, self.theta)
        o = self.attention(q, k, v, self.scale, self.cap_a, self.layer_window(i))
        a = o.reshape(T, self.nH * self.d) @ t[p + "self_attn.o_proj.weight"].T
        if taps is not None:
            taps[f"layer{i}.attn_out"] = a
        x = x + rms_norm(a, t[p + "post_attention_layernorm.weight"], self.eps)
        n = rms_norm(x, t[p + "pre_feedforward_layernorm.weight"], self.eps)
        f = geglu(n, t[p + "mlp.gate_proj.weight"], t[p + "mlp.up_proj.weight"],
                  t[p + "mlp.down_proj.weight"])
        x = x + rms_norm(f, t[p + "post_feedforward_layernorm.weight"], self.eps)
        if taps is not None:
            taps[f"layer{i}.out"] = x
        return x

    def forward(self, tokens, taps=None) -> torch.Tensor:
        """Logits [T, V] of one whole sequence.  llama3.rs:13632-14614."""
        T = len(tokens)
        positions = torch.arange(T, device=self.device)
        x = self.embed(tokens)
        for i in range(self.L):
            x = self.layer(i, x, positions, taps)
        n = rms_norm(x, self.t["model.norm.weight"], self.eps)
        head = self.t.get("lm_head.weight", self.t["model.embed_tokens.weight"])
        return softcap(n @ head.T, self.cap_f)      # llama3.rs:14590-14611

    def greedy(self, prompt, n_new, stop_ids=()):
        """Greedy continuation by re-running the whole sequence each step; lowest index on ties."""
        seq = list(prompt)
        out = []
        for _ in range(n_new):
            logits = self.forward(seq)[-1]
            nxt = int(torch.argmax(logits))
            if nxt in stop_ids:
                break
            out.append(nxt)
            seq.append(nxt)
        return out


# --------------------------------------------------------------------------- sampling

def plain_softmax(x: torch.Tensor) -> torch.Tensor:
    """Subtract the maximum, exp, divide by the sum.  src/sampling.rs:77-92."""
    e = torch.exp(x - x.max())
    return e / e.sum()


def plain_top_k(logits: torch.Tensor, k: int) -> torch.Tensor:
    """Keep the k largest, ties at the threshold kept; k = 0 or k >= len: no-op.  src/sampling.rs:25-41."""
    if k == 0 or k >= logits.numel():
        return logits
    thr = torch.sort(logits, descending=True).values[k - 1]
    return torch.where(logits < thr, torch.full_like(logits, float("-inf")), logits)


def plain_top_p(logits: torch.Tensor, p: float) -> torch.Tensor:
    """Keep the shortest descending prefix whose cumulative probability exceeds p.  src/sampling.rs:45-74."""
    if p >= 1.0:
        return logits
    probs = plain_softmax(logits)
    order = torch.argsort(probs, descending=True, stable=True)
    cum = 0.0
    keep = []
    for idx in order.tolist():
        keep.append(idx)
        cum += float(probs[idx])
        if cum > p:
            break
    out = torch.full_like(logits, float("-inf"))
    out[keep] = logits[keep]
    return out


def plain_inverse_cdf(probs: torch.Tensor, u: float) -> int:
    """First i with u < sum_{j<=i} p_j, else the last index.  src/sampling.rs:114-123."""
    cum = 0.0
    for i, p in enumerate(probs.tolist()):
        cum += p
        if u < cum:
            return i
    return probs.numel() - 1


def plain_sample(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, u: float) -> int:
    """temperature -> top-k -> (top-p) -> softmax -> inverse CDF; T < 1e-6 is greedy.

    examples/generate_gpu.rs:122-129 for the order and the greedy threshold.
    """
    if temperature < 1e-6:
        return int(torch.argmax(logits))
    x = logits / temperature
    x = plain_top_k(x, top_k)
    x = plain_top_p(x, top_p)
    return plain_inverse_cdf(plain_softmax(x), u)
