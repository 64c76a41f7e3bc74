"""Pins of the plain implementation by what fixes it beside the reference's text: vectors that the
reference's own tests hold, special cases that reduce to a library routine, and invariants, each
chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place, an off-by-one
window) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from helpers import TINY_A, TINY_B, model_folder, plain_model, random_tokens
from plain import gemma2_plain as P

D = torch.float64


# ------------------------------------------------------------------ RMSNorm
def test_rms_norm_reference_vector():
    # llama3.rs:20482-20498: x = [1,2,3,4], unit weight (here w = 0 under the 1 + w convention), eps 1e-5
    x = torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=D)
    out = P.rms_norm(x, torch.zeros(4, dtype=D), 1e-5)
    assert torch.allclose(out, x / math.sqrt(7.5 + 1e-5), atol=1e-12)
    # integration_tests.rs:521-538: constant vectors come out near 1
    assert torch.allclose(P.rms_norm(torch.ones(4, dtype=D), torch.zeros(4, dtype=D), 1e-6), torch.ones(4, dtype=D), atol=1e-5)
    assert torch.allclose(P.rms_norm(torch.full((2,), 2.0, dtype=D), torch.zeros(2, dtype=D), 1e-6), torch.ones(2, dtype=D), atol=1e-5)


def test_rms_norm_is_library_rms_norm_with_one_plus_w():
    torch.manual_seed(0)
    x, w = torch.randn(5, 24, dtype=D), torch.randn(24, dtype=D) * 0.1
    assert torch.allclose(P.rms_norm(x, w, 1e-5), F.rms_norm(x, (24,), weight=1 + w, eps=1e-5), atol=1e-12)
    # the weight is an offset from one: w = 0 gives unit RMS, not zero
    y = P.rms_norm(x, torch.zeros(24, dtype=D), 1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=D), atol=1e-6)
    # scale invariance up to eps
    assert torch.allclose(P.rms_norm(7 * x, w, 1e-12), P.rms_norm(x, w, 1e-12), atol=1e-9)


# ------------------------------------------------------------------ rotation
def test_rope_identity_norm_and_complex_form():
    torch.manual_seed(1)
    x = torch.randn(7, 3, 24, dtype=D)
    pos = torch.tensor([0, 5, 5, 17, 100, 1000, 8191])
    y = P.rope_half_split(x, pos, 500000.0)
    assert torch.allclose(y[0], x[0], atol=1e-15)                               # llama3.rs:20510-20518
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-12)           # llama3.rs:20520-20528
    # pairs (j, j + d/2) as complex numbers times e^{i pos f_j}: a wrong pairing (2j, 2j+1) or sign fails
    half = 12
    f = 500000.0 ** (-2.0 * torch.arange(half, dtype=D) / 24)
    z = torch.complex(x[..., :half], x[..., half:]) * torch.polar(torch.ones(7, half, dtype=D), pos[:, None].to(D) * f)[:, None, :]
    assert torch.allclose(y, torch.cat([z.real, z.imag], dim=-1), atol=1e-12)


def test_rope_scores_depend_on_distance_only():
    torch.manual_seed(2)
    q, k = torch.randn(1, 1, 16, dtype=D), torch.randn(1, 1, 16, dtype=D)
    def score(m, n):
        return (P.rope_half_split(q, torch.tensor([m]), 1e4) * P.rope_half_split(k, torch.tensor([n]), 1e4)).sum()
    assert abs(score(9, 4) - score(109, 104)) < 1e-10
    assert abs(score(9, 4) - score(4, 9)) > 1e-3           # and on its sign
    a = P.rope_half_split(P.rope_half_split(q, torch.tensor([3]), 1e4), torch.tensor([4]), 1e4)
    assert torch.allclose(a, P.rope_half_split(q, torch.tensor([7]), 1e4), atol=1e-12)


# ------------------------------------------------------------------ attention
def _qkv(T, nH, nKV, d, seed):
    torch.manual_seed(seed)
    return torch.randn(T, nH, d, dtype=D), torch.randn(T, nKV, d, dtype=D), torch.randn(T, nKV, d, dtype=D)


def test_attention_reduces_to_library_sdpa_without_cap_and_window():
    q, k, v = _qkv(11, 6, 3, 24, 3)
    scale = 32 ** -0.5
    ours = P.attention_core(q, k, v, scale, None, None)
    lib = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.repeat_interleave(2, 1).transpose(0, 1)[None],
                                         v.repeat_interleave(2, 1).transpose(0, 1)[None], is_causal=True, scale=scale)
    assert torch.allclose(ours, lib[0].transpose(0, 1), atol=1e-12)
    assert torch.allclose(P.attention_core(q, k, v, scale, None, 11), ours, atol=1e-14)      # W >= T is global


def test_attention_loop_and_dense_forms_agree_with_cap_and_window():
    q, k, v = _qkv(19, 4, 1, 16, 4)
    for cap, win in ((50.0, 8), (2.0, 6), (None, 3), (1.5, None), (5.0, 1)):
        a = P.attention_core(q * 3, k * 3, v, 0.25, cap, win)
        b = P.attention_dense(q * 3, k * 3, v, 0.25, cap, win)
        assert torch.allclose(a, b, atol=1e-12), (cap, win)


def test_attention_window_edge():
    # W keys, the query's own included (llama3.rs:5444-5451): position p reads p+1-W .. p
    q, k, v = _qkv(12, 2, 1, 8, 5)
    W, p = 4, 9
    base = P.attention_core(q, k, v, 0.3, 10.0, W)[p]
    k2, v2 = k.clone(), v.clone()
    k2[p - W] += 5.0; v2[p - W] += 5.0                      # just outside: p - W
    assert torch.equal(P.attention_core(q, k2, v2, 0.3, 10.0, W)[p], base)
    k3, v3 = k.clone(), v.clone()
    v3[p + 1 - W] += 5.0                                    # the oldest key inside
    assert (P.attention_core(q, k3, v3, 0.3, 10.0, W)[p] - base).abs().max() > 1e-3
    # window 1: only itself, output is its own value
    assert torch.allclose(P.attention_core(q, k, v, 0.3, 10.0, 1)[p, 0], v[p, 0], atol=1e-14)


def test_attention_invariants():
    q, k, v = _qkv(9, 4, 2, 8, 6)
    out = P.attention_core(q, k, v, 0.35, 7.0, None)
    # causal: the first row attends to itself only (integration_tests.rs:187-201)
    assert torch.allclose(out[0, 0], v[0, 0], atol=1e-14) and torch.allclose(out[0, 3], v[0, 1], atol=1e-14)
    # prefix invariance: later tokens change nothing earlier
    k2, v2 = k.clone(), v.clone(); k2[6:] += 1; v2[6:] -= 1
    assert torch.equal(P.attention_core(q, k2, v2, 0.35, 7.0, None)[:6], out[:6])
    # grouped heads: consecutive query heads share a kv head (h // g), so equal queries give equal outputs
    q2 = q.clone(); q2[:, 1] = q2[:, 0]; q2[:, 2] = q2[:, 0]
    o2 = P.attention_core(q2, k, v, 0.35, 7.0, None)
    assert torch.allclose(o2[:, 0], o2[:, 1], atol=1e-14) and not torch.allclose(o2[:, 0], o2[:, 2], atol=1e-3)
    # the cap comes before the softmax: huge scores saturate to +-cap, leaving a spread of at most 2 cap
    big = P.attention_core(q * 1e4, k, v, 1.0, 0.5, None)
    uniformish = v[:, 0].cumsum(0) / torch.arange(1, 10, dtype=D)[:, None]
    assert (big[:, 0] - uniformish).abs().max() < 0.9 * v.abs().max()


def test_online_softmax_vector_of_the_reference():
    # llama3.rs:20398-20479: closed-form q, k, v, d = 8, T = 5; two-pass softmax, scale 1/sqrt(8)
    d, T = 8, 5
    q = torch.tensor([i * 0.11 - 0.4 for i in range(d)], dtype=D)
    k = torch.tensor([[math.sin((t + 1) * 0.07 - e * 0.03) for e in range(d)] for t in range(T)], dtype=D)
    v = torch.tensor([[math.cos((t + 3) * 0.13 + e * 0.05) for e in range(d)] for t in range(T)], dtype=D)
    s = (k @ q) / math.sqrt(d)
    expect = torch.softmax(s, 0) @ v
    qq = torch.zeros(T, 1, d, dtype=D); qq[T - 1, 0] = q
    got = P.attention_core(qq, k[:, None, :], v[:, None, :], 1 / math.sqrt(d), None, None)[T - 1, 0]
    assert torch.allclose(got, expect, atol=1e-12)


# ------------------------------------------------------------------ softcap, GELU
def test_softcap_properties():
    x = torch.linspace(-200, 200, 401, dtype=D)
    y = P.softcap(x, 30.0)
    assert torch.allclose(y, -P.softcap(-x, 30.0)) and (y.abs() < 30).all() and (y[1:] >= y[:-1]).all()
    assert abs(float(P.softcap(torch.tensor(0.01, dtype=D), 30.0)) - 0.01) < 1e-9
    assert P.softcap(x, None) is x


def test_gelu_is_the_tanh_form():
    x = torch.linspace(-6, 6, 97, dtype=D)
    assert torch.allclose(P.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-12)
    assert (P.gelu_tanh(x) - F.gelu(x)).abs().max() > 1e-4                       # not the erf form
    g = P.gelu_tanh(torch.tensor([0.0, 1.0, -3.0, 1.0, 2.0, 3.0], dtype=D))     # integration_tests.rs:564-587
    assert g[0] == 0 and g[1] > 0.5 and abs(g[2]) < 0.01 and g[3] < g[4] < g[5]
    x2, wg, wu, wd = torch.randn(3, 8, dtype=D), torch.randn(12, 8, dtype=D), torch.randn(12, 8, dtype=D), torch.randn(8, 12, dtype=D)
    assert torch.allclose(P.geglu(x2, wg, wu, wd), F.linear(F.gelu(F.linear(x2, wg), approximate="tanh") * F.linear(x2, wu), wd), atol=1e-12)


# ------------------------------------------------------------------ whole model
def small_plain(L, W, H=32, seed=0, **over):
    """A plain model of L layers from a configuration and random tensors made here."""
    cfg = dict(vocab_size=50, hidden_size=H, num_hidden_layers=L, num_attention_heads=2, num_key_value_heads=1, head_dim=8,
               intermediate_size=48, rope_theta=100.0, rms_norm_eps=1e-6, sliding_window=W, attn_logit_softcapping=50.0,
               final_logit_softcapping=30.0, query_pre_attn_scalar=8)
    cfg.update(over)
    g = torch.Generator().manual_seed(seed)
    r = lambda *shape, std=0.3: torch.randn(*shape, generator=g, dtype=D) * std
    t = {"model.embed_tokens.weight": r(cfg["vocab_size"], H), "model.norm.weight": r(H, std=0.1)}
    for i in range(L):
        p = f"model.layers.{i}."
        t[p + "self_attn.q_proj.weight"], t[p + "self_attn.o_proj.weight"] = r(16, H), r(H, 16)
        t[p + "self_attn.k_proj.weight"], t[p + "self_attn.v_proj.weight"] = r(8, H), r(8, H)
        t[p + "mlp.gate_proj.weight"], t[p + "mlp.up_proj.weight"], t[p + "mlp.down_proj.weight"] = r(48, H), r(48, H), r(H, 48)
        for n in ("input", "post_attention", "pre_feedforward", "post_feedforward"):
            t[p + n + "_layernorm.weight"] = r(H, std=0.1)
    return P.PlainGemma2(cfg, t)


def test_which_layers_slide():
    """Layer 0 slides and layer 1 is global (llama3.rs:4634-4641).  With one layer, nothing before the window can
    reach a position; with two, it does, and only through layer 1.  The mistake this catches: the kinds swapped
    (odd layers sliding), or every layer of one kind."""
    W, T, p = 4, 14, 13
    toks = random_tokens(50, T, 1)
    far = list(toks); far[p - W] = (toks[p - W] + 1) % 50          # the newest token outside position p's window
    edge = list(toks); edge[p + 1 - W] = (toks[p + 1 - W] + 1) % 50  # the oldest inside it
    one = small_plain(1, W)
    assert torch.equal(one.forward(far)[p], one.forward(toks)[p])        # layer 0 slides: bit-equal
    assert (one.forward(edge)[p] - one.forward(toks)[p]).abs().max() > 1e-6
    two = small_plain(2, W)
    assert (two.forward(far)[p] - two.forward(toks)[p]).abs().max() > 1e-6      # layer 1 sees everything
    # only through layer 1: the far token reaches p in layer 1 directly, so layer 0's output at p is still bit-equal
    taps_a, taps_b = {}, {}
    two.forward(far, taps_a); two.forward(toks, taps_b)
    assert torch.equal(taps_a["layer0.out"][p], taps_b["layer0.out"][p])
    assert not torch.equal(taps_a["layer1.attn_out"][p], taps_b["layer1.attn_out"][p])
    # with three layers the third slides again: a token two windows back reaches p only through layer 1
    three = small_plain(3, W)
    assert [three.layer_window(i) for i in range(3)] == [W, None, W]


def test_scale_comes_before_the_cap():
    """score * scale, then cap * tanh(. / cap) (llama3.rs:5622-5642).  With cap 0.01 and scale 100 the capped scores
    lie within +-0.01 whatever the scale, so the softmax is nearly uniform; in the other order (cap, then scale)
    they spread over +-1 and it is not."""
    q, k, v = _qkv(10, 2, 1, 8, 8)
    for form in (P.attention_core, P.attention_dense):
        out = form(q, k, v, 100.0, 0.01, None)
        uniform = v[:, 0].cumsum(0) / torch.arange(1, 11, dtype=D)[:, None]
        assert (out[:, 0] - uniform).abs().max() < 0.03 * v.abs().max()
    raw = torch.einsum("td,ud->tu", q[:, 0], k[:, 0])
    swapped = (0.01 * torch.tanh(raw / 0.01)) * 100.0                    # the mistake
    swapped = swapped.masked_fill(torch.arange(10)[None, :] > torch.arange(10)[:, None], float("-inf"))
    assert (torch.softmax(swapped, -1) @ v[:, 0] - uniform).abs().max() > 4 * 0.03 * v.abs().max()


def test_the_head_is_the_embedding_matrix():
    """One matrix serves the embedding and the head (llama3.rs:12896-12906): doubling row v doubles logit v
    before the cap and nothing else, for sequences without token v; and changes every logit of a sequence that
    holds token v, because its input changed.  The mistake this catches: a head with a matrix of its own."""
    m = small_plain(2, 4)
    v = 17
    toks = [t for t in random_tokens(50, 12, 2) if t != v]
    base = m.forward(toks)
    m2 = small_plain(2, 4)
    m2.t["model.embed_tokens.weight"][v] *= 2.0
    out = m2.forward(toks)
    others = [i for i in range(50) if i != v]
    assert torch.equal(out[:, others], base[:, others])
    precap = lambda z: 30.0 * torch.atanh(z / 30.0)
    assert torch.allclose(precap(out[:, v]), 2.0 * precap(base[:, v]), atol=1e-9)
    with_v = toks[:5] + [v] + toks[5:]
    assert (m2.forward(with_v)[6:, others] - m.forward(with_v)[6:, others]).abs().max() > 1e-6


def test_embedding_scale_is_the_square_root_taken_in_f32():
    """x = E[token] * sqrt(width), the root taken of the width as an f32 (llama3.rs:13697-13703).  For a width of
    96 that is 9.797959327697754, not the 64-bit root 9.797958971132712; no factor on the way out."""
    m = small_plain(1, 4, H=96)
    E = m.t["model.embed_tokens.weight"]
    assert torch.equal(m.embed([5, 9]), E[[5, 9]] * 9.797959327697754)
    assert not torch.equal(m.embed([5]), E[[5]] * math.sqrt(96.0))
    assert torch.equal(small_plain(1, 4, H=64).embed([3]), small_plain(1, 4, H=64).t["model.embed_tokens.weight"][[3]] * 8.0)


@pytest.mark.parametrize("name", ["tiny-a", "tiny-b"])
def test_model_invariants(name):
    m = plain_model(model_folder(name, "float32"))
    toks = random_tokens(m.V, 20, 3)
    full = m.forward(toks)
    assert full.shape == (20, m.V)
    assert torch.allclose(m.forward(toks[:13]), full[:13], atol=1e-12)           # prefix invariance
    # the final cap bites where logits are large: the hot variant's logits come near the cap and stay below it,
    # and without the cap they pass it
    hot = plain_model(model_folder(name, "float32", hot=12.0))
    capped = hot.forward(toks)
    assert 0.4 * hot.cap_f < capped.abs().max() < hot.cap_f
    hot.cap_f = None
    assert hot.forward(toks).abs().max() > capped.abs().max() + 0.5


def test_model_layer_kinds_and_norm_places():
    folder = model_folder("tiny-b", "float32")
    m = plain_model(folder)
    toks = random_tokens(m.V, 16, 4)
    base = m.forward(toks)
    m2 = plain_model(folder); m2.window = 1000
    assert (m2.forward(toks)[-1] - base[-1]).abs().max() > 1e-9                 # the window matters at T=16 > 6
    assert torch.allclose(m2.forward(toks)[:6], base[:6], atol=1e-12)           # and not before it bites
    # post norms act on the branch before the add: zeroing a post norm's (1 + w) removes the branch
    m3 = plain_model(folder)
    for i in range(3):
        m3.t[f"model.layers.{i}.post_attention_layernorm.weight"].fill_(-1.0)
        m3.t[f"model.layers.{i}.post_feedforward_layernorm.weight"].fill_(-1.0)
    x = m3.embed(toks)
    out = x
    for i in range(3):
        out = m3.layer(i, out, torch.arange(16))
    assert torch.allclose(out, x, atol=1e-12)


# ------------------------------------------------------------------ sampling
def test_sampling_vectors_of_the_reference():
    T = torch.tensor
    assert int(torch.argmax(T([1.0, 5.0, 3.0]))) == 1                                     # integration_tests.rs:358-466
    assert int(torch.argmax(T([0.7, 0.5, 0.7, 0.3]))) == 0                                # llama3.rs:21263-21269
    p = T([0.1, 0.2, 0.7])
    assert [P.plain_inverse_cdf(p, u) for u in (0.05, 0.25, 0.95)] == [0, 1, 2]
    assert [P.plain_inverse_cdf(T([0.5, 0.5]), u) for u in (0.0, 0.49, 0.51)] == [0, 0, 1]
    assert torch.allclose(P.plain_softmax(T([0.0, 0.0, 0.0])), torch.full((3,), 1 / 3))
    assert torch.allclose(P.plain_softmax(T([1000.0, 1000.0, 0.0])), T([0.5, 0.5, 0.0]))
    x = T([1.0, 4.0, 2.0, 3.0])
    assert torch.equal(P.plain_top_k(x, 0), x) and torch.equal(P.plain_top_k(x, 9), x)
    assert P.plain_top_k(x, 2).tolist() == [float("-inf"), 4.0, float("-inf"), 3.0]
    assert P.plain_top_k(T([1.0, 3.0, 3.0, 0.0]), 1).tolist()[1:3] == [3.0, 3.0]         # ties at the threshold kept
    kept = P.plain_top_p(T([0.0, math.log(2.0), math.log(7.0)]), 0.75)                     # probs .1 .2 .7
    assert kept.tolist()[0] == float("-inf") and kept.tolist()[1] != float("-inf")
    assert P.plain_sample(x, 0.0, 0, 1.0, 0.3) == 1 and P.plain_sample(x, 1e-3, 0, 1.0, 0.99) == 1
