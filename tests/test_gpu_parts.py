"""Each part alone against its plain formula, built directly from its registry with sizes that no
model here uses, and a toy architecture whose mixer keeps state of its own: registered, built,
loaded with random weights and stepped without touching the package's files."""
import math
from dataclasses import dataclass

import pytest
import torch
import torch.nn.functional as F

import alice_llm_amd as alice
from alice_llm_amd.cache import Cache
from alice_llm_amd.config.plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from alice_llm_amd.engine.model import CausalLM
from alice_llm_amd.engine.step import Engine
from alice_llm_amd.hip import ops
from alice_llm_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, CacheNeed, ParamSpec, Part, Precision,
                                 ResidualStream, StateNeed)
from alice_llm_amd.weights.loader import init_random
from helpers import TOL
from plain import gemma2_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"
D = torch.float64
PRECS = ["float32", "bfloat16"]


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def tol(prec):
    return 2e-5 if prec == "float32" else 3e-2


@pytest.mark.parametrize("prec", PRECS)
def test_norm_part_and_stream_fusion(prec):
    p = Precision.of(prec)
    H, T = 136, 6
    n1 = NORMS.get("rmsnorm")(p, dim=H, eps=3e-6, weight_offset=1.0)
    n2 = NORMS.get("rmsnorm")(p, dim=H, eps=1e-5, weight_offset=0.0)
    w1, w2 = rnd(H, seed=1, scale=0.1, dtype=torch.bfloat16), rnd(H, seed=2, dtype=torch.bfloat16)
    n1.assign("weight", w1); n2.assign("weight", w2)
    x0, br = rnd(T, H, seed=3, scale=2.0), rnd(T, H, seed=4)
    s = ResidualStream(x0.clone(), p)
    first = s.normed(n1)
    assert first.dtype == p.act
    ref_first = P.rms_norm(x0.double(), w1.double(), 3e-6)
    assert (first.double() - ref_first).abs().max() < tol(prec)
    s.push(br, n2)
    second = s.normed(n1)                                      # add of the normed branch and the next norm, fused
    xr = x0.double() + br.double() * torch.rsqrt((br.double() ** 2).mean(-1, keepdim=True) + 1e-5) * w2.double()
    assert (s.x.double() - xr).abs().max() < 1e-5
    assert (second.double() - P.rms_norm(xr, w1.double(), 3e-6)).abs().max() < tol(prec)
    s.push(br, None)
    rows = torch.tensor([5, 1], dtype=torch.int32, device=DEV)
    last = s.rows_normed(n2, rows)
    xr2 = xr + br.double()
    want = xr2[[5, 1]] * torch.rsqrt((xr2[[5, 1]] ** 2).mean(-1, keepdim=True) + 1e-5) * w2.double()
    assert (last.double() - want).abs().max() < tol(prec) * 4


@pytest.mark.parametrize("prec", PRECS)
def test_gated_mlp_part(prec):
    p = Precision.of(prec)
    H, I, T = 96, 208, 9
    ff = FEED_FORWARDS.get("gated_mlp")(p, hidden_size=H, intermediate_size=I, activation="gelu_tanh")
    assert {k: v.shape for k, v in ff.param_specs().items()} == {"gate_proj.weight": (I, H), "up_proj.weight": (I, H), "down_proj.weight": (H, I)}
    ws = {n: rnd(*s.shape, seed=i, scale=0.2, dtype=torch.bfloat16) for i, (n, s) in enumerate(ff.param_specs().items())}
    for n, w in ws.items():
        ff.assign(n, w)
    ff.finalize()
    x = rnd(T, H, seed=9, dtype=p.act)
    out = ff.forward(x, None)
    out = out.sum(0) if out.dim() == 3 else out
    ref = P.geglu(x.double(), ws["gate_proj.weight"].double(), ws["up_proj.weight"].double(), ws["down_proj.weight"].double())
    assert out.dtype == torch.float32 and (out.double() - ref).abs().max() < tol(prec) * max(1.0, float(ref.abs().max()))
    with pytest.raises(ValueError, match="activation"):
        FEED_FORWARDS.get("gated_mlp")(p, hidden_size=H, intermediate_size=I, activation="relu6")


@dataclass
class _Ctx:
    tokens: torch.Tensor
    positions: torch.Tensor
    seq_of_token: torch.Tensor
    slots: torch.Tensor
    max_position: int
    is_decode: bool = False
    want_rows: torch.Tensor = None
    n_tokens: int = 0
    n_seqs: int = 1
    max_new: int = 0
    max_context: int = 0
    cu_seqlens: torch.Tensor = None
    context_lens: torch.Tensor = None
    new_lens: tuple = ()
    start_lens: tuple = ()
    slot_ids: tuple = ()


def make_ctx(starts, news):
    pos = [s + i for s, n in zip(starts, news) for i in range(n)]
    seq = [b for b, n in enumerate(news) for _ in range(n)]
    cu = [0]
    for n in news:
        cu.append(cu[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return _Ctx(tokens=i32([0] * len(pos)), positions=i32(pos), seq_of_token=i32(seq), slots=i32(list(range(len(news)))),
                max_position=max(pos), is_decode=all(n == 1 for n in news), n_tokens=len(pos), n_seqs=len(news),
                max_new=max(news), max_context=max(s + n for s, n in zip(starts, news)), cu_seqlens=i32(cu),
                context_lens=i32([s + n for s, n in zip(starts, news)]), new_lens=tuple(news), start_lens=tuple(starts),
                slot_ids=tuple(range(len(news))))


@pytest.mark.parametrize("prec", PRECS)
@pytest.mark.parametrize("nH,nKV,d,window,cap,rotary", [(4, 2, 32, None, None, 32), (3, 1, 48, 20, 8.0, 48), (2, 2, 16, 70, 3.0, 8)])
def test_attention_part_alone_in_two_steps(prec, nH, nKV, d, window, cap, rotary):
    """The mixer on a cache of its own: a prompt step, then single tokens, against the plain formulas;
    also a position encoding with a rotated width below the head size."""
    p = Precision.of(prec)
    H, T = 80, 90
    rope = POSITIONS.get("rope")(p, DEV, dim=d, theta=3000.0, max_positions=128, rotary_dim=rotary)
    att = MIXERS.get("attention")(p, {"r": rope}, hidden_size=H, num_heads=nH, num_kv_heads=nKV, head_dim=d,
                                  scale=0.21, softcap=cap, window=window, position="r")
    ws = {n: rnd(*s.shape, seed=10 + i, scale=0.15, dtype=torch.bfloat16) for i, (n, s) in enumerate(att.param_specs().items())}
    for n, w in ws.items():
        att.assign(n, w)
    att.finalize()
    need = att.cache_need()
    assert need.kv.num_kv_heads == nKV and need.kv.head_dim == d and need.kv.window == window
    cache = Cache([need], max_tokens=128, dtype=p.act, device=DEV, max_seqs=1)
    slot = cache.open()
    x = rnd(T, H, seed=20, dtype=p.act)
    xd = x.double().cpu()
    ws = {n: w.cpu() for n, w in ws.items()}
    q = (xd @ ws["q_proj.weight"].double().T).view(T, nH, d)
    k = (xd @ ws["k_proj.weight"].double().T).view(T, nKV, d)
    v = (xd @ ws["v_proj.weight"].double().T).view(T, nKV, d)
    pos = torch.arange(T)
    rot = lambda a: torch.cat([P.rope_half_split(a[..., :rotary], pos, 3000.0), a[..., rotary:]], -1)
    ref = P.attention_core(rot(q), rot(k), v, 0.21, cap, window).reshape(T, nH * d) @ ws["o_proj.weight"].double().T
    got = []
    for start, n in ((0, 70), (70, 1), (71, 1), (72, 18)):
        cache.reserve([slot], [n])
        bt = torch.tensor(cache.block_table_rows(0, [slot], 2), dtype=torch.int32, device=DEV)
        out = att.forward(x[start:start + n].contiguous(), make_ctx([start], [n]), cache.view(0, [bt]))
        got.append(out.sum(0) if out.dim() == 3 else out)
        cache.commit([slot], [n])
    got = torch.cat(got)
    assert (got.double().cpu() - ref.cpu()).abs().max() < tol(prec) * max(1.0, float(ref.abs().max()))


# ------------------------------------------------------------------ a toy architecture
class ToyDecayMixer(Part):
    """A mixer with state of its own and no keys: s <- a * s + x W_in per token, output s W_out.  State is a
    fixed-size vector per sequence, advanced token by token inside a step (a sequential scan in torch: this
    is a test of the interfaces, not a kernel)."""

    def __init__(self, precision, positions, *, hidden_size, state_size, decay):
        self.p, self.H, self.S, self.decay = precision, hidden_size, state_size, decay
        self.w = {}

    def param_specs(self):
        return {"in.weight": ParamSpec((self.S, self.H), 0.1), "out.weight": ParamSpec((self.H, self.S), 0.1)}

    def assign(self, name, t):
        self.w[name] = t.float()

    def cache_need(self):
        return CacheNeed(state=StateNeed("s", (self.S,), torch.float32))

    def forward(self, x, ctx, cache):
        u = x.float() @ self.w["in.weight"].T
        out = torch.empty_like(u)
        row = 0
        state = cache.state["s"]
        for slot, n in zip(ctx.slot_ids, ctx.new_lens):
            s = state[slot]
            for i in range(n):
                s = self.decay * s + u[row]
                out[row] = s
                row += 1
            state[slot] = s
        return (out @ self.w["out.weight"].T).contiguous()


class ToyMLP(Part):
    def __init__(self, precision, *, hidden_size):
        self.H = hidden_size

    def param_specs(self):
        return {"w.weight": ParamSpec((self.H, self.H), 0.1)}

    def assign(self, name, t):
        self.w = t.float()

    def forward(self, x, ctx):
        return torch.relu(x.float() @ self.w.T).contiguous()


class ToyConfig:
    def __init__(self, d):
        self.d = dict(d)
        self.torch_dtype = "bfloat16"

    @classmethod
    def from_dict(cls, d):
        return cls(d)

    def to_dict(self):
        return dict(self.d)

    def plan(self):
        H, V, L = self.d["width"], self.d["vocab"], self.d["depth"]
        norm = lambda name: PartSpec("rmsnorm", {"dim": H, "eps": 1e-5, "weight_offset": 0.0}, name)
        layers = []
        for i in range(L):
            toy = i % 2 == 0      # toy mixer on even layers, windowed attention on odd ones: one model, two mixers
            mixer = (PartSpec("toy_decay", {"hidden_size": H, "state_size": self.d["state"], "decay": 0.5}, "mix") if toy else
                     PartSpec("attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "scale": 0.25,
                                            "window": 5, "position": "rope"}, "attn"))
            layers.append(LayerPlan(block="prenorm", mixer=mixer, feed_forward=PartSpec("toy_mlp", {"hidden_size": H}, "ff"),
                                    norms={"pre_mixer": norm("n1"), "pre_ff": norm("n2")}, prefix=f"blocks.{i}."))
        # the schedule runs layer 0 twice (each run with state of its own), and layer 3 reads the cache that
        # the run of layer 1 (entry 1) wrote
        schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(2), ScheduleEntry(3, cache_from=1)]
        return ModelPlan(vocab_size=V, hidden_size=H, max_positions=256,
                         embedding=PartSpec("embedding", {"vocab_size": V, "dim": H, "scale": 1.0}, "emb"),
                         positions={"rope": PartSpec("rope", {"dim": 16, "theta": 100.0, "max_positions": 256})},
                         layers=tuple(layers), schedule=tuple(schedule[:L + 1] if L >= 4 else schedule[:3]),
                         final_norm=norm("final"), head=PartSpec("lm_head", {"vocab_size": V, "dim": H, "tied_to": "emb"}, "head"))


def toy_plain(model, tokens):
    """The toy model for one whole sequence in 64-bit, from the loaded tensors."""
    lm = model.lm
    get = lambda part: part.weight.double().cpu() if hasattr(part, "weight") else None
    E = lm.embedding.table.weight.double().cpu()
    x = E[torch.tensor(tokens)]
    T = len(tokens)
    rms = lambda v, n: v * torch.rsqrt((v * v).mean(-1, keepdim=True) + n.eps) * (n.weight_offset + n.weight.double().cpu())
    kv_seen = {}
    for ei, e in enumerate(lm.plan.schedule):
        layer = lm.layers[e.layer]
        h = rms(x, layer.norms["pre_mixer"])
        m = layer.mixer
        if isinstance(m, ToyDecayMixer):
            u = h @ m.w["in.weight"].double().cpu().T
            s = torch.zeros(m.S, dtype=D)           # every run of the schedule has state of its own
            outs = []
            for i in range(T):
                s = 0.5 * s + u[i]
                outs.append(s)
            a = torch.stack(outs) @ m.w["out.weight"].double().cpu().T
        else:
            W = m.qkv.weight.double().cpu()
            order = m.position.projection_row_order(2, 1, 16)     # the fused rows may be in the rotation's pair order
            if m.pair_order:
                W = torch.empty_like(W).index_copy_(0, order, W)
            q = (h @ W[:32].T).view(T, 2, 16)
            if e.cache_from is None:
                k = P.rope_half_split((h @ W[32:48].T).view(T, 1, 16), torch.arange(T), 100.0)
                v = (h @ W[48:64].T).view(T, 1, 16)
                kv_seen[ei] = (k, v)
            else:
                k, v = kv_seen[e.cache_from]
            o = P.attention_core(P.rope_half_split(q, torch.arange(T), 100.0), k, v, 0.25, None, 5)
            a = o.reshape(T, 32) @ m.o.weight.double().cpu().T
        x = x + a
        h = rms(x, layer.norms["pre_ff"])
        x = x + torch.relu(h @ layer.feed_forward.w.double().cpu().T)
    return rms(x, lm.final_norm) @ E.T


def test_toy_architecture_with_a_stateful_mixer_registers_builds_and_steps():
    MIXERS.register("toy_decay", ToyDecayMixer)
    FEED_FORWARDS.register("toy_mlp", ToyMLP)
    alice.register_architecture("ToyForCausalLM", ToyConfig)
    raw = {"architectures": ["ToyForCausalLM"], "width": 48, "vocab": 77, "depth": 4, "state": 24}
    assert "ToyForCausalLM" in alice.registered_architectures()
    # float32 weights stay row-major, which the toy's 64-bit replica reads directly
    model = alice.Model.random(raw, seed=3, dtype="float32", stored_dtype=torch.float32)
    assert list(model.lm.param_specs())[:3] == ["emb.weight", "blocks.0.mix.in.weight", "blocks.0.mix.out.weight"]
    eng = model.engine(max_tokens=256, max_seqs=3)
    assert [g.layers for g in eng.cache.groups] == [[1]] and sorted(eng.cache.state) == [0, 2, 3]   # by schedule entry
    seqs = [[5, 9, 3, 70, 1, 22, 8, 8, 41, 60, 2, 13], [7, 7, 30], [11, 2, 64, 19, 50, 6]]
    # cut-up runs of the engine against its own whole runs, and both against the 64-bit replica
    slots = eng.open(3)
    whole = eng.step(slots, seqs, "all")
    eng.close(slots)
    slots = eng.open(3)
    parts = [eng.step(slots, [s[:2] for s in seqs], "all")]
    left = [s[2:] for s in seqs]
    live = [0, 1, 2]
    outs = {i: [] for i in live}
    while live:
        lg = eng.step([slots[i] for i in live], [[left[i].pop(0)] for i in live], "last")
        for row, i in enumerate(live):
            outs[i].append(lg[row])
        done = [i for i in live if not left[i]]
        eng.close([slots[i] for i in done])                    # state of a closed slot is zeroed when it is taken again
        live = [i for i in live if i not in done]
    first = parts[0]
    cut = torch.cat([torch.cat([first[2 * i:2 * i + 2], torch.stack(outs[i])]) for i in range(3)])
    assert (cut - whole).abs().max() < 1e-5
    ref = torch.cat([toy_plain(model, t) for t in seqs])
    assert (whole.double().cpu() - ref).abs().max() < 2e-5 * max(1.0, float(ref.abs().max()))
    # slots used again start from zero state: the same requests give the same logits
    slots = eng.open(3)
    assert torch.equal(eng.step(slots, seqs, "all"), whole)
    eng.close(slots)
    eng.cache.check_consistent()


def test_toy_architecture_against_its_plain_replica():
    MIXERS.register("toy_decay", ToyDecayMixer)
    FEED_FORWARDS.register("toy_mlp", ToyMLP)
    alice.register_architecture("ToyForCausalLM", ToyConfig)
    raw = {"architectures": ["ToyForCausalLM"], "width": 48, "vocab": 77, "depth": 4, "state": 24}
    model = alice.Model.random(raw, seed=4, dtype="float32", stored_dtype=torch.float32)
    eng = model.engine(max_tokens=128, max_seqs=2)
    toks = [5, 9, 3, 70, 1, 22, 8, 8, 41, 60, 2, 13, 0, 76]
    s = eng.open(1)
    got = torch.cat([eng.step(s, [toks[:9]], "all")] + [eng.step(s, [[t]], "last") for t in toks[9:]])
    ref = toy_plain(model, toks)
    assert (got.double().cpu() - ref).abs().max() < 2e-5 * max(1.0, float(ref.abs().max()))


# ------------------------------------------------------------------ a toy with two state tensors, in captured steps
class ToyTailScanMixer(Part):
    """A mixer with two state tensors per sequence, of different shapes: the last two inputs (a convolution's
    tail) and a running sum.  c_t = u_t + 0.5 u_(t-1) + 0.25 u_(t-2) with u = x W_in, s_t = decay * s_(t-1) + c_t,
    output s_t W_out.  Single-token steps index the state with ctx.slots on the device and launch the same
    kernels whatever the batch holds, so the mixer declares graph_safe and its decode steps are captured into
    HIP graphs; prompts loop on the host."""
    graph_safe = True

    def __init__(self, precision, positions, *, hidden_size, state_size, decay):
        self.H, self.S, self.decay = hidden_size, state_size, decay
        self.w = {}

    def param_specs(self):
        return {"in.weight": ParamSpec((self.S, self.H), 0.1), "out.weight": ParamSpec((self.H, self.S), 0.1)}

    def assign(self, name, t):
        self.w[name] = t.float()

    def cache_need(self):
        return CacheNeed(state=(StateNeed("tail", (2, self.S)), StateNeed("sum", (self.S,))))

    def forward(self, x, ctx, cache):
        u = x.float() @ self.w["in.weight"].T
        tail, acc = cache.state["tail"], cache.state["sum"]
        if ctx.is_decode:
            idx = ctx.slots.long()                             # device data: the same launches for any batch
            t = tail.index_select(0, idx)                      # [B, 2, S]: u_(t-2), u_(t-1)
            s = self.decay * acc.index_select(0, idx) + u + 0.5 * t[:, 1] + 0.25 * t[:, 0]
            acc.index_copy_(0, idx, s)
            tail.index_copy_(0, idx, torch.stack([t[:, 1], u], dim=1))
            out = s
        else:
            assert not ctx.captured
            out = torch.empty_like(u)
            row = 0
            for slot, n in zip(ctx.slot_ids, ctx.new_lens):
                t2, t1, s = tail[slot, 0].clone(), tail[slot, 1].clone(), acc[slot].clone()
                for _ in range(n):
                    s = self.decay * s + u[row] + 0.5 * t1 + 0.25 * t2
                    out[row] = s
                    t2, t1 = t1, u[row]
                    row += 1
                tail[slot, 0], tail[slot, 1], acc[slot] = t2, t1, s
        return (out @ self.w["out.weight"].T).contiguous()


class ToyGraphMLP(ToyMLP):
    graph_safe = True


class ToyScanConfig(ToyConfig):
    def plan(self):
        H, V = self.d["width"], self.d["vocab"]
        norm = lambda name: PartSpec("rmsnorm", {"dim": H, "eps": 1e-5, "weight_offset": 0.0}, name)
        scan = lambda: PartSpec("toy_tail_scan", {"hidden_size": H, "state_size": self.d["state"], "decay": 0.75}, "mix")
        att = PartSpec("attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "scale": 0.25,
                                     "window": 7, "position": "rope"}, "attn")
        layers = [LayerPlan(block="prenorm", mixer=m, feed_forward=PartSpec("toy_graph_mlp", {"hidden_size": H}, "ff"),
                            norms={"pre_mixer": norm("n1"), "pre_ff": norm("n2")}, prefix=f"blocks.{i}.")
                  for i, m in enumerate([scan(), att, scan()])]
        return ModelPlan(vocab_size=V, hidden_size=H, max_positions=256,
                         embedding=PartSpec("embedding", {"vocab_size": V, "dim": H, "scale": 1.0}, "emb"),
                         positions={"rope": PartSpec("rope", {"dim": 16, "theta": 100.0, "max_positions": 256})},
                         layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(3)),
                         final_norm=norm("final"), head=PartSpec("lm_head", {"vocab_size": V, "dim": H, "tied_to": "emb"}, "head"))


def toy_scan_plain(model, tokens):
    E = model.lm.embedding.table.weight.double().cpu()
    return _toy_scan_plain_from(model, E[torch.tensor(tokens)], E)


def _toy_scan_plain_from(model, x, E):
    lm = model.lm
    T = x.shape[0]
    rms = lambda v, n: v * torch.rsqrt((v * v).mean(-1, keepdim=True) + n.eps) * (n.weight_offset + n.weight.double().cpu())
    for layer in lm.layers:
        h = rms(x, layer.norms["pre_mixer"])
        m = layer.mixer
        if isinstance(m, ToyTailScanMixer):
            u = h @ m.w["in.weight"].double().cpu().T
            s, outs = torch.zeros(m.S, dtype=D), []
            for i in range(T):
                s = 0.75 * s + u[i] + (0.5 * u[i - 1] if i >= 1 else 0) + (0.25 * u[i - 2] if i >= 2 else 0)
                outs.append(s)
            a = torch.stack(outs) @ m.w["out.weight"].double().cpu().T
        else:
            W = m.qkv.weight.double().cpu()
            if m.pair_order:
                W = torch.empty_like(W).index_copy_(0, m.position.projection_row_order(2, 1, 16), W)
            pos = torch.arange(T)
            q, k, v = (h @ W[:32].T).view(T, 2, 16), (h @ W[32:48].T).view(T, 1, 16), (h @ W[48:64].T).view(T, 1, 16)
            o = P.attention_core(P.rope_half_split(q, pos, 100.0), P.rope_half_split(k, pos, 100.0), v, 0.25, None, 7)
            a = o.reshape(T, 32) @ m.o.weight.double().cpu().T
        x = x + a
        x = x + torch.relu(rms(x, layer.norms["pre_ff"]) @ layer.feed_forward.w.double().cpu().T)
    return rms(x, lm.final_norm) @ E.T


def test_toy_mixer_with_two_state_tensors_runs_in_captured_steps():
    MIXERS.register("toy_tail_scan", ToyTailScanMixer)
    FEED_FORWARDS.register("toy_graph_mlp", ToyGraphMLP)
    alice.register_architecture("ToyScanForCausalLM", ToyScanConfig)
    raw = {"architectures": ["ToyScanForCausalLM"], "width": 48, "vocab": 83, "state": 20}
    model = alice.Model.random(raw, seed=6, dtype="float32", stored_dtype=torch.float32)
    graph = model.engine(max_tokens=64 * 6, max_seqs=5)
    eager = model.engine(max_tokens=64 * 6, max_seqs=5, use_graphs=False)
    assert graph.use_graphs and not eager.use_graphs            # state does not turn captured steps off
    assert sorted(graph.cache.state) == [0, 2] and set(graph.cache.state[0]) == {"tail", "sum"}
    assert graph.cache.state[0]["tail"].shape == (5 + 1, 2, 20)   # a row per slot and the spare one
    g = torch.Generator().manual_seed(9)
    seqs = [torch.randint(0, 83, (n,), generator=g).tolist() for n in (30, 12, 21)]
    prompt = [4, 1, 9]
    refs = [toy_scan_plain(model, t) for t in seqs]
    for again in range(2):                                       # a second batch on the same slots: state starts at zero
        got = {}
        for eng in (graph, eager):
            slots = eng.open(3)
            first = eng.step(slots, [s[:n] for s, n in zip(seqs, prompt)], "all")
            outs, o = {}, 0
            for i, n in enumerate(prompt):
                outs[i] = [first[o:o + n]]
                o += n
            live, step = [0, 1, 2], 0
            while live:                                           # three rows in a captured step of four: one padded row
                lg = eng.step([slots[i] for i in live], [[seqs[i][prompt[i] + step]] for i in live], "last")
                for row, i in enumerate(live):
                    outs[i].append(lg[row:row + 1].clone())
                step += 1
                done = [i for i in live if prompt[i] + step >= len(seqs[i])]
                eng.close([slots[i] for i in done])
                live = [i for i in live if i not in done]
            got[eng] = [torch.cat(outs[i]) for i in range(3)]
            eng.cache.check_consistent()
        for i in range(3):
            assert (got[graph][i].double().cpu() - refs[i]).abs().max() < 2e-5 * max(1.0, float(refs[i].abs().max())), (again, i)
            assert (got[graph][i] - got[eager][i]).abs().max() < 1e-5
    assert len(graph._graphs) >= 3                               # batches of 3 (a bucket of 4), 2 and 1


class ToyTailScanDeviceMixer(ToyTailScanMixer):
    """The same mixer with its steps of several tokens on the device as well: a scan over the step's longest
    piece whose rows come from ctx.cu_seqlens, with sequences that have ended masked out.  It therefore declares
    graph_safe_prompts, and short prompt steps of its model are recorded into HIP graphs like the built-in parts'."""
    graph_safe_prompts = True

    def forward(self, x, ctx, cache):
        if ctx.is_decode:
            return super().forward(x, ctx, cache)
        u = x.float() @ self.w["in.weight"].T
        tail, acc = cache.state["tail"], cache.state["sum"]
        T = u.shape[0]
        idx, cu = ctx.slots.long(), ctx.cu_seqlens.long()
        held = tail.index_select(0, idx)
        t2, t1, s = held[:, 0], held[:, 1], acc.index_select(0, idx)
        u_pad = torch.cat([u, torch.zeros_like(u[:1])])
        out = torch.zeros_like(u_pad)                            # row T takes what ended sequences write
        dump = torch.full_like(cu[:-1], T)
        for t in range(ctx.max_new):                             # a host constant of the (captured) step
            rows = cu[:-1] + t
            live = rows < cu[1:]
            rows = torch.where(live, rows, dump)
            ut = u_pad.index_select(0, rows)
            lv = live[:, None]
            s = torch.where(lv, self.decay * s + ut + 0.5 * t1 + 0.25 * t2, s)
            t2, t1 = torch.where(lv, t1, t2), torch.where(lv, ut, t1)
            out.index_copy_(0, rows, s)
        acc.index_copy_(0, idx, s)
        tail.index_copy_(0, idx, torch.stack([t2, t1], dim=1))
        return (out[:T] @ self.w["out.weight"].T).contiguous()


class ToyLearnedPositions(alice.parts.embedding.Embedding):
    """An embedding that adds a learned row per position: it needs the step's positions, which it finds in ctx."""

    def __init__(self, precision, *, vocab_size, dim, max_positions, scale=1.0):
        super().__init__(precision, vocab_size=vocab_size, dim=dim, scale=scale)
        self.P = max_positions

    def param_specs(self):
        return {**super().param_specs(), "positions.weight": ParamSpec((self.P, self.dim), 0.3)}

    def assign(self, name, t):
        if name == "positions.weight":
            self.pos = t.float()
        else:
            super().assign(name, t)

    def forward(self, ctx):
        return super().forward(ctx) + self.pos.index_select(0, ctx.positions.long())


class ToyScanDeviceConfig(ToyScanConfig):
    def plan(self):
        import dataclasses
        plan = super().plan()
        swap = lambda m: PartSpec("toy_tail_scan_device", m.args, m.name) if m.kind == "toy_tail_scan" else m
        layers = tuple(dataclasses.replace(l, mixer=swap(l.mixer)) for l in plan.layers)
        emb = PartSpec("toy_learned_positions", {"vocab_size": plan.vocab_size, "dim": plan.hidden_size, "max_positions": 256}, "emb")
        return dataclasses.replace(plan, layers=layers, embedding=emb)


def test_toy_embedding_reads_positions_and_stateful_prompt_steps_are_captured():
    """An embedding that needs the step's positions and a stateful mixer that advances its state on the device in
    steps of several tokens: registered from here; the engine then records short prompt steps of this model too,
    and a recorded step gives what the eager one and the plain replica give."""
    from alice_llm_amd.parts import EMBEDDINGS
    MIXERS.register("toy_tail_scan", ToyTailScanMixer)
    MIXERS.register("toy_tail_scan_device", ToyTailScanDeviceMixer)
    FEED_FORWARDS.register("toy_graph_mlp", ToyGraphMLP)
    EMBEDDINGS.register("toy_learned_positions", ToyLearnedPositions)
    alice.register_architecture("ToyScanDeviceForCausalLM", ToyScanDeviceConfig)
    alice.register_architecture("ToyScanForCausalLM", ToyScanConfig)
    raw = {"architectures": ["ToyScanDeviceForCausalLM"], "width": 48, "vocab": 83, "state": 20}
    model = alice.Model.random(raw, seed=8, dtype="float32", stored_dtype=torch.float32)
    assert "emb.positions.weight" in model.lm.param_specs()
    graph = model.engine(max_tokens=64 * 6, max_seqs=4)
    eager = model.engine(max_tokens=64 * 6, max_seqs=4, use_graphs=False)
    assert graph.capture_prompts and not eager.capture_prompts
    host_only = alice.Model.random(dict(raw, architectures=["ToyScanForCausalLM"]), seed=8, dtype="float32", stored_dtype=torch.float32)
    assert not host_only.engine(max_tokens=64).capture_prompts        # its prompts loop on the host: not recorded

    def plain(tokens):                                                # the replica of the scan toy plus the position rows
        lm = model.lm
        E, Ppos = lm.embedding.table.weight.double().cpu(), lm.embedding.pos.double().cpu()
        return _toy_scan_plain_from(model, E[torch.tensor(tokens)] + Ppos[:len(tokens)], E)

    g = torch.Generator().manual_seed(10)
    seqs = [torch.randint(0, 83, (n,), generator=g).tolist() for n in (29, 17, 23)]
    refs = [plain(t) for t in seqs]
    for again in range(3):                                            # the third pass replays what the second recorded
        got = {}
        for eng in (graph, eager):
            slots = eng.open(3)
            rows = {i: [] for i in range(3)}
            at = [0, 0, 0]
            for piece in ((5, 2, 7), (6, 6, 1), (3, 4, 9)):           # pieces of prompts, last rows wanted: 14, 13, 16 tokens
                lg = eng.step(slots, [seqs[i][at[i]:at[i] + n] for i, n in enumerate(piece)], "last")
                for i, n in enumerate(piece):
                    at[i] += n
                    rows[i].append((at[i] - 1, lg[i].clone()))
            live = [0, 1, 2]
            while live:
                lg = eng.step([slots[i] for i in live], [[seqs[i][at[i]]] for i in live], "last")
                for r, i in enumerate(live):
                    rows[i].append((at[i], lg[r].clone()))
                    at[i] += 1
                done = [i for i in live if at[i] >= len(seqs[i])]
                eng.close([slots[i] for i in done])
                live = [i for i in live if i not in done]
            got[eng] = rows
            eng.cache.check_consistent()
        for i in range(3):
            for (p, a), (p2, b) in zip(got[graph][i], got[eager][i]):
                assert p == p2 and (a - b).abs().max() < 1e-5, (again, i, p)
                assert (a.double().cpu() - refs[i][p]).abs().max() < 2e-5 * max(1.0, float(refs[i].abs().max())), (again, i, p)
    assert len(graph._prompt_graphs) >= 2                             # token counts 14, 13 and 16 round to 16: two shapes (with and without padding)


class ToyF32KeyMixer(Part):
    """One head of plain causal attention, in torch, that keeps its keys and values in 32-bit whatever the run's
    activation dtype is: it says so in its KVNeed, and the cache gives its layers pages of their own in that dtype."""

    def __init__(self, precision, positions, *, hidden_size, head_dim):
        self.H, self.d = hidden_size, head_dim
        self.w = {}

    def param_specs(self):
        return {f"{n}.weight": ParamSpec((self.d, self.H), 0.2) for n in "qkv"} | {"o.weight": ParamSpec((self.H, self.d), 0.2)}

    def assign(self, name, t):
        self.w[name] = t.float()

    def cache_need(self):
        from alice_llm_amd.parts import KVNeed
        return CacheNeed(kv=KVNeed(1, self.d, dtype=torch.float32))

    def forward(self, x, ctx, cache):
        assert cache.k.dtype == torch.float32 and cache.v.dtype == torch.float32
        x = x.float()
        q, k, v = (x @ self.w[f"{n}.weight"].T for n in "qkv")
        P_ = cache.k.shape[2]
        pos, seq = ctx.positions.long(), ctx.seq_of_token.long()
        page = cache.block_table.long()[seq, pos // P_]
        cache.k[page, 0, pos % P_] = k
        cache.v[page, 0, pos % P_] = v
        out = torch.empty_like(q)
        row = 0
        for b, (start, n) in enumerate(zip(ctx.start_lens, ctx.new_lens)):
            pages = cache.block_table[b, :-(-(start + n) // P_)].long()
            keys, vals = cache.k[pages, 0].reshape(-1, self.d)[:start + n], cache.v[pages, 0].reshape(-1, self.d)[:start + n]
            sc = (q[row:row + n] @ keys.T) * self.d ** -0.5
            mask = torch.arange(start + n, device=x.device)[None, :] > (start + torch.arange(n, device=x.device))[:, None]
            out[row:row + n] = torch.softmax(sc.masked_fill(mask, float("-inf")), -1) @ vals
            row += n
        return (out @ self.w["o.weight"].T).contiguous()


class ToyMixedKeysConfig(ToyConfig):
    def plan(self):
        H, V = self.d["width"], self.d["vocab"]
        norm = lambda name: PartSpec("rmsnorm", {"dim": H, "eps": 1e-5, "weight_offset": 0.0}, name)
        mixers = [PartSpec("toy_f32_keys", {"hidden_size": H, "head_dim": 24}, "mix"),
                  PartSpec("attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "scale": 0.25,
                                         "position": "rope"}, "attn")]
        layers = [LayerPlan(block="prenorm", mixer=m, feed_forward=PartSpec("toy_mlp", {"hidden_size": H}, "ff"),
                            norms={"pre_mixer": norm("n1"), "pre_ff": norm("n2")}, prefix=f"blocks.{i}.") for i, m in enumerate(mixers)]
        return ModelPlan(vocab_size=V, hidden_size=H, max_positions=256,
                         embedding=PartSpec("embedding", {"vocab_size": V, "dim": H, "scale": 1.0}, "emb"),
                         positions={"rope": PartSpec("rope", {"dim": 16, "theta": 100.0, "max_positions": 256})},
                         layers=tuple(layers), schedule=(ScheduleEntry(0), ScheduleEntry(1)),
                         final_norm=norm("final"), head=PartSpec("lm_head", {"vocab_size": V, "dim": H, "tied_to": "emb"}, "head"))


def test_toy_mixer_keeps_32_bit_keys_under_bfloat16_activations():
    """A mixer names the dtype of its pages in its KVNeed: in a bfloat16 run its layers get 32-bit pages of their
    own beside the built-in attention's bfloat16 pages, and what they hold was never rounded."""
    MIXERS.register("toy_f32_keys", ToyF32KeyMixer)
    FEED_FORWARDS.register("toy_mlp", ToyMLP)
    alice.register_architecture("ToyMixedKeysForCausalLM", ToyMixedKeysConfig)
    raw = {"architectures": ["ToyMixedKeysForCausalLM"], "width": 64, "vocab": 71}
    model = alice.Model.random(raw, seed=9, dtype="bfloat16")
    eng = model.engine(max_tokens=256, max_seqs=2)
    assert sorted((g.layers, g.k.dtype, g.need.head_dim) for g in eng.cache.groups) == \
        [([0], torch.float32, 24), ([1], torch.bfloat16, 16)]
    assert not eng.use_graphs                                    # the toy loops on the host
    seqs = [[5, 9, 3, 70, 1, 22, 8, 8, 41, 60, 2, 13, 44, 6], [7, 7, 30, 12]]
    slots = eng.open(2)
    whole = eng.step(slots, seqs, "all")
    # the first layer's pages hold its keys to the last bit: x W_k in 32-bit of the normed embedding rows
    lm, m = model.lm, model.lm.layers[0].mixer
    from types import SimpleNamespace
    toks = torch.tensor(seqs[0] + seqs[1], dtype=torch.int32, device=DEV)      # the step's rows, so that the product is the same call
    x0 = lm.embedding.forward(SimpleNamespace(tokens=toks))
    h = lm.layers[0].norms["pre_mixer"].forward(x0, torch.bfloat16)
    page = eng.cache.groups[[g.layers for g in eng.cache.groups].index([0])]
    held = page.k[0, page.table(slots[0])[0], 0, :len(seqs[0])]
    assert torch.equal(held, (h.float() @ m.w["k.weight"].T)[:len(seqs[0])]) and not torch.equal(held, held.bfloat16().float())
    eng.close(slots)
    # cut into steps, the shorter request ending earlier: the same logits within bfloat16 rounding
    slots = eng.open(2)
    first = eng.step(slots, [s[:3] for s in seqs], "all")
    outs = {0: [first[:3]], 1: [first[3:]]}
    for i in range(3, len(seqs[0])):
        live = [b for b in (0, 1) if i < len(seqs[b])]
        lg = eng.step([slots[b] for b in live], [[seqs[b][i]] for b in live], "last")
        for row, b in enumerate(live):
            outs[b].append(lg[row:row + 1])
        if i + 1 == len(seqs[1]):
            eng.close([slots[1]])
    eng.close([slots[0]])
    cut = torch.cat([torch.cat(outs[0]), torch.cat(outs[1])])
    assert (cut - whole).abs().max() < 3e-2 * max(1.0, float(whole.abs().max()))
    eng.cache.check_consistent()
    # two runs that share a cache must agree on its dtype
    import dataclasses
    bad = dataclasses.replace(model.lm.plan, schedule=(ScheduleEntry(0), ScheduleEntry(1, cache_from=0)))
    with pytest.raises(ValueError, match="cannot read the cache"):
        CausalLM(bad, "bfloat16", DEV)


# ------------------------------------------------------------------ a second toy: routing and another position encoding
class ToyRoutedFF(Part):
    """A feed-forward with routing: router logits in 32-bit, the two best of E experts per token, their
    softmax weights, experts y = relu(x W1_e^T) W2_e^T.  In torch: a test of the interface (a feed-forward sees
    x and the step's context, nothing else), not a kernel."""

    def __init__(self, precision, *, hidden_size, inner, experts):
        self.H, self.I, self.E = hidden_size, inner, experts
        self.w = {}

    def param_specs(self):
        specs = {"router.weight": ParamSpec((self.E, self.H), 0.5)}
        for e in range(self.E):
            specs[f"experts.{e}.up.weight"] = ParamSpec((self.I, self.H), 0.1)
            specs[f"experts.{e}.down.weight"] = ParamSpec((self.H, self.I), 0.1)
        return specs

    def assign(self, name, t):
        self.w[name] = t.float()

    @staticmethod
    def route(x, w, E, I, H, dtype):
        logits = x.to(dtype) @ w["router.weight"].to(dtype).T
        top, idx = logits.topk(2, dim=-1)
        gate = torch.softmax(top, dim=-1)
        out = torch.zeros(x.shape[0], H, dtype=dtype, device=x.device)
        for e in range(E):
            for slot in range(2):
                rows = (idx[:, slot] == e).nonzero().flatten()
                if rows.numel():
                    h = torch.relu(x[rows].to(dtype) @ w[f"experts.{e}.up.weight"].to(dtype).T)
                    out[rows] += gate[rows, slot, None] * (h @ w[f"experts.{e}.down.weight"].to(dtype).T)
        return out, idx

    def forward(self, x, ctx):
        out, self.last_choice = self.route(x, self.w, self.E, self.I, self.H, torch.float32)
        return out.contiguous()


class ToyInterleavedRotation(Part):
    """Another position encoding: rotation of the pairs (2j, 2j + 1) (the reference's other pairing,
    llama3.rs:5323-5336), done in torch; keys and values then go into the cache through the library's write
    without rotation.  What a position encoding owes the attention mixer is rotate_and_store, nothing more."""

    def __init__(self, precision, device, *, dim, theta, max_positions):
        j = torch.arange(dim // 2, dtype=torch.float64)
        ang = torch.arange(max_positions, dtype=torch.float64)[:, None] * theta ** (-2.0 * j / dim)
        self.cos, self.sin = torch.cos(ang).float().to(device), torch.sin(ang).float().to(device)
        self.none = POSITIONS.get("none")(precision, device)

    def rotate(self, x, positions):            # x: [T, heads, d]
        c, s = self.cos[positions.long()][:, None, :].to(x.dtype), self.sin[positions.long()][:, None, :].to(x.dtype)
        a, b = x[..., 0::2], x[..., 1::2]
        return torch.stack([a * c - b * s, a * s + b * c], dim=-1).flatten(-2)

    def rotate_and_store(self, qkv, q_out, ctx, cache, *, num_heads, num_kv_heads, head_dim, kv_layout=0):
        T = qkv.shape[0]
        nq, nk = num_heads * head_dim, num_kv_heads * head_dim
        rot = qkv.clone()
        rot[:, :nq] = self.rotate(qkv[:, :nq].float().view(T, num_heads, head_dim), ctx.positions).reshape(T, nq).to(qkv.dtype)
        rot[:, nq:nq + nk] = self.rotate(qkv[:, nq:nq + nk].float().view(T, num_kv_heads, head_dim), ctx.positions).reshape(T, nk).to(qkv.dtype)
        self.none.rotate_and_store(rot, q_out, ctx, cache, num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim,
                                   kv_layout=kv_layout)


class ToyRoutedConfig(ToyConfig):
    def plan(self):
        H, V = self.d["width"], self.d["vocab"]
        norm = lambda name: PartSpec("rmsnorm", {"dim": H, "eps": 1e-5, "weight_offset": 0.0}, name)
        att = lambda: PartSpec("attention", {"hidden_size": H, "num_heads": 3, "num_kv_heads": 3, "head_dim": 16, "scale": 0.25,
                                             "position": "twist"}, "attn")
        ffs = [PartSpec("toy_routed", {"hidden_size": H, "inner": 40, "experts": 3}, "moe"), PartSpec("toy_mlp", {"hidden_size": H}, "ff")]
        layers = [LayerPlan(block="prenorm", mixer=att(), feed_forward=ffs[i % 2], norms={"pre_mixer": norm("n1"), "pre_ff": norm("n2")},
                            prefix=f"blocks.{i}.") for i in range(self.d["depth"])]
        return ModelPlan(vocab_size=V, hidden_size=H, max_positions=128,
                         embedding=PartSpec("embedding", {"vocab_size": V, "dim": H, "scale": 1.0}, "emb"),
                         positions={"twist": PartSpec("toy_interleaved", {"dim": 16, "theta": 50.0, "max_positions": 128})},
                         layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(self.d["depth"])),
                         final_norm=norm("final"), head=PartSpec("lm_head", {"vocab_size": V, "dim": H, "tied_to": "emb"}, "head"))


def toy_routed_plain(model, tokens):
    lm = model.lm
    E = lm.embedding.table.weight.double().cpu()
    x = E[torch.tensor(tokens)]
    T = len(tokens)
    rms = lambda v, n: v * torch.rsqrt((v * v).mean(-1, keepdim=True) + n.eps) * (n.weight_offset + n.weight.double().cpu())
    pos = torch.arange(T)
    ang = pos.double()[:, None] * 50.0 ** (-2.0 * torch.arange(8, dtype=D) / 16)
    def twist(v):        # [T, heads, 16], pairs (2j, 2j+1)
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        a, b = v[..., 0::2], v[..., 1::2]
        return torch.stack([a * c - b * s, a * s + b * c], dim=-1).flatten(-2)
    choices = []
    for layer in lm.layers:
        h = rms(x, layer.norms["pre_mixer"])
        W = layer.mixer.qkv.weight.double().cpu()
        q, k, v = (h @ W[:48].T).view(T, 3, 16), (h @ W[48:96].T).view(T, 3, 16), (h @ W[96:].T).view(T, 3, 16)
        o = P.attention_core(twist(q), twist(k), v, 0.25, None, None)
        x = x + o.reshape(T, 48) @ layer.mixer.o.weight.double().cpu().T
        h = rms(x, layer.norms["pre_ff"])
        ff = layer.feed_forward
        if isinstance(ff, ToyRoutedFF):
            y, idx = ToyRoutedFF.route(h, {k_: v_.cpu() for k_, v_ in ff.w.items()}, ff.E, ff.I, ff.H, D)
            choices.append(idx)
            x = x + y
        else:
            x = x + torch.relu(h @ ff.w.double().cpu().T)
    return rms(x, lm.final_norm) @ E.T, choices


def test_toy_architecture_with_routing_and_another_position_encoding():
    FEED_FORWARDS.register("toy_mlp", ToyMLP)
    FEED_FORWARDS.register("toy_routed", ToyRoutedFF)
    POSITIONS.register("toy_interleaved", ToyInterleavedRotation)
    alice.register_architecture("ToyRoutedForCausalLM", ToyRoutedConfig)
    raw = {"architectures": ["ToyRoutedForCausalLM"], "width": 48, "vocab": 61, "depth": 3}
    model = alice.Model.random(raw, seed=5, dtype="float32", stored_dtype=torch.float32)
    assert "blocks.0.moe.experts.2.down.weight" in model.lm.param_specs() and "blocks.1.ff.w.weight" in model.lm.param_specs()
    eng = model.engine(max_tokens=256, max_seqs=2)
    seqs = [[5, 9, 3, 60, 1, 22, 8, 8, 41, 2, 13, 0, 33, 17], [7, 7, 30, 12, 55]]
    slots = eng.open(2)
    whole = eng.step(slots, seqs, "all")
    eng.close(slots)
    refs = [toy_routed_plain(model, t) for t in seqs]
    ref = torch.cat([r[0] for r in refs])
    assert (whole.double().cpu() - ref).abs().max() < 2e-5 * max(1.0, float(ref.abs().max()))
    # the routing really spreads tokens over the experts (else the test would not see a wrong choice)
    assert len(set(torch.cat([c.flatten() for c in refs[0][1]]).tolist())) == 3
    # cut into steps, in a batch whose shorter request ends earlier: the same logits
    slots = eng.open(2)
    first = eng.step(slots, [s[:3] for s in seqs], "all")
    outs = {0: [first[:3]], 1: [first[3:]]}
    for i in range(3, len(seqs[0])):
        live = [b for b in (0, 1) if i < len(seqs[b])]
        lg = eng.step([slots[b] for b in live], [[seqs[b][i]] for b in live], "last")
        for row, b in enumerate(live):
            outs[b].append(lg[row:row + 1])
        if i + 1 == len(seqs[1]):
            eng.close([slots[1]])
    eng.close([slots[0]])
    cut = torch.cat([torch.cat(outs[0]), torch.cat(outs[1])])
    assert (cut - whole).abs().max() < 1e-5
    eng.cache.check_consistent()


class ToyDistanceBiasConfig(ToyConfig):
    """Positions known to the scores alone: attention without rotation whose heads subtract slope * distance (one
    slope a head, a constructor argument of the attention mixer), global and windowed layers in turn."""
    SLOPES = (0.5, 0.125, 0.03125, 0.0)

    def plan(self):
        H, V = self.d["width"], self.d["vocab"]
        norm = lambda name: PartSpec("rmsnorm", {"dim": H, "eps": 1e-5, "weight_offset": 0.0}, name)
        att = lambda i: PartSpec("attention", {"hidden_size": H, "num_heads": 4, "num_kv_heads": 2, "head_dim": self.d["head"],
                                               "scale": 0.2, "softcap": 4.0 if i % 2 else None, "window": 6 if i % 2 else None,
                                               "position": "none", "score_bias_slopes": self.SLOPES}, "attn")
        layers = [LayerPlan(block="prenorm", mixer=att(i), feed_forward=PartSpec("toy_graph_mlp", {"hidden_size": H}, "ff"),
                            norms={"pre_mixer": norm("n1"), "pre_ff": norm("n2")}, prefix=f"blocks.{i}.") for i in range(self.d["depth"])]
        return ModelPlan(vocab_size=V, hidden_size=H, max_positions=128,
                         embedding=PartSpec("embedding", {"vocab_size": V, "dim": H, "scale": 1.0}, "emb"), positions={},
                         layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(self.d["depth"])),
                         final_norm=norm("final"), head=PartSpec("lm_head", {"vocab_size": V, "dim": H, "tied_to": "emb"}, "head"))


def toy_distance_bias_plain(raw, tensors, tokens):
    """Whole sequence in 64-bit from the stored tensors (by name), dense attention with the distance term."""
    H, d = raw["width"], raw["head"]
    w = lambda name: tensors[name].double().cpu()
    E = w("emb.weight")
    x = E[torch.tensor(tokens)]
    T = len(tokens)
    rms = lambda v, g: v * torch.rsqrt((v * v).mean(-1, keepdim=True) + 1e-5) * g
    ar = torch.arange(T)
    dist = (ar[None, :] - ar[:, None]).double()
    for i in range(raw["depth"]):
        pre = f"blocks.{i}."
        h = rms(x, w(pre + "n1.weight"))
        q, k, v = ((h @ w(pre + f"attn.{n}_proj.weight").T).view(T, -1, d) for n in "qkv")
        cap, window = (4.0, 6) if i % 2 else (None, None)
        heads = []
        for hd in range(4):
            sc = (q[:, hd] @ k[:, hd // 2].T) * 0.2
            if cap:
                sc = cap * torch.tanh(sc / cap)
            sc = sc + ToyDistanceBiasConfig.SLOPES[hd] * dist
            seen = (dist <= 0) & ((dist > -window) if window else (dist <= 0))
            heads.append(torch.softmax(sc.masked_fill(~seen, float("-inf")), -1) @ v[:, hd // 2])
        x = x + torch.stack(heads, 1).reshape(T, 4 * d) @ w(pre + "attn.o_proj.weight").T
        h = rms(x, w(pre + "n2.weight"))
        x = x + torch.relu(h @ w(pre + "ff.w.weight").T)
    return rms(x, w("final.weight")) @ E.T


@pytest.mark.parametrize("dtype,head", [("float32", 16), ("bfloat16", 16), ("bfloat16", 64)])
def test_toy_architecture_with_a_position_term_at_the_score_stage(dtype, head):
    """Another kind of position encoding, registered from here: no rotation, a distance term in the scores.  It is a
    parameter of the attention mixer (score_bias_slopes), so the toy needs no mixer and no kernel of its own; with
    it the mixer keeps its cache row-major and takes the 32-bit attention kernel, also where the head size (64)
    would otherwise go to the matrix cores.  Whole prompts, then single tokens through captured steps, against a
    64-bit replica that reads the stored tensors; without the term the logits differ by far more than the bound."""
    from alice_llm_amd.engine.model import CausalLM
    from alice_llm_amd.weights.loader import random_tensors
    from helpers import model_from_tensors
    FEED_FORWARDS.register("toy_graph_mlp", ToyGraphMLP)
    alice.register_architecture("ToyDistanceBiasForCausalLM", ToyDistanceBiasConfig)
    raw = {"architectures": ["ToyDistanceBiasForCausalLM"], "width": 64, "vocab": 83, "depth": 3, "head": head}
    cfg = alice.config_from_dict(raw)
    stored = torch.float32 if dtype == "float32" else torch.bfloat16
    tensors = dict(random_tensors(CausalLM(cfg.plan(), "float32", "cpu").param_specs(), 9, stored, DEV))
    for k in tensors:                                           # norm weights about 1 and matrices of 0.12: logits and scores of order 1
        if "proj.weight" in k or k == "emb.weight":
            tensors[k] = (tensors[k].float() * 6.0).to(stored)
        elif k.endswith(("n1.weight", "n2.weight", "final.weight")):
            tensors[k] = (tensors[k].float() + 1.0).to(stored)
    model = model_from_tensors(cfg, tensors, dtype)
    mixers = [l.mixer for l in model.lm.layers]
    assert all(m.kv_layout == ops.KV_ROW and m._slopes is not None for m in mixers)
    seqs = [[5, 9, 3, 60, 1, 22, 8, 8, 41, 2, 13, 0, 33, 17, 70, 4, 4, 29], [7, 7, 30, 12, 55, 81, 2]]
    refs = [toy_distance_bias_plain(raw, tensors, t) for t in seqs]
    assert max(float(r.abs().max()) for r in refs) > 2.0
    tol = (2e-5 if dtype == "float32" else 4e-2) * max(1.0, max(float(r.abs().max()) for r in refs))
    eng = model.engine(max_tokens=256, max_seqs=2)
    slots = eng.open(2)
    whole = eng.step(slots, seqs, "all")
    eng.close(slots)
    assert (whole.double().cpu() - torch.cat(refs)).abs().max() < tol
    for again in range(3):                                      # the third pass replays captured single-token steps
        slots = eng.open(2)
        got = {0: [], 1: []}
        first = eng.step(slots, [s[:4] for s in seqs], "last")
        for i in range(4, len(seqs[0])):
            live = [b for b in (0, 1) if i < len(seqs[b])]
            lg = eng.step([slots[b] for b in live], [[seqs[b][i]] for b in live], "last")
            for row, b in enumerate(live):
                got[b].append(lg[row].clone())
            if i + 1 == len(seqs[1]):
                eng.close([slots[1]])
        eng.close([slots[0]])
        for b in (0, 1):
            assert (first[b].double().cpu() - refs[b][3]).abs().max() < tol
            assert (torch.stack(got[b]).double().cpu() - refs[b][4:]).abs().max() < tol, (again, b)
    assert eng.use_graphs and len(eng._graphs) >= 1
    # the term matters: the same tensors without it are far from the replica
    for m in mixers:
        m._slopes = None
    slots = eng.open(2)
    flat = eng.step(slots, seqs, "all")
    eng.close(slots)
    assert (flat.double().cpu() - torch.cat(refs)).abs().max() > 10 * tol
    eng.cache.check_consistent()


@pytest.mark.parametrize("prec", PRECS)
def test_embedding_and_tied_head_parts(prec):
    from alice_llm_amd.parts import EMBEDDINGS, HEADS
    p = Precision.of(prec)
    V, H = 203, 72
    emb = EMBEDDINGS.get("embedding")(p, vocab_size=V, dim=H, scale=2.5)
    head = HEADS.get("lm_head")(p, vocab_size=V, dim=H, softcap=4.0, tied_to="emb")
    assert head.param_specs() == {} and emb.param_specs()["weight"].shape == (V, H)
    E = rnd(V, H, seed=30, scale=0.3, dtype=torch.bfloat16)
    emb.assign("weight", E)
    emb.finalize(); head.finalize(); head.tie(emb)
    tok = torch.tensor([0, 202, 17, 17], dtype=torch.int32, device=DEV)
    from types import SimpleNamespace
    x = emb.forward(SimpleNamespace(tokens=tok))
    assert x.dtype == torch.float32 and (x.double() - E.double()[tok.long()] * 2.5).abs().max() < 1e-6
    n = rnd(5, H, seed=31, dtype=p.act)
    logits = head.forward(n)
    ref = 4.0 * torch.tanh((n.double() @ E.double().T) / 4.0)
    assert logits.dtype == torch.float32 and (logits.double() - ref).abs().max() < tol(prec)
    untied = HEADS.get("lm_head")(p, vocab_size=V, dim=H, softcap=None, tied_to=None)
    assert untied.param_specs()["weight"].shape == (V, H)
    untied.assign("weight", E)
    assert (untied.forward(n).double() - n.double() @ E.double().T).abs().max() < tol(prec) * 3


def test_rotary_part_table_is_accurate_far_out():
    p = Precision.of("float32")
    rope = POSITIONS.get("rope")(p, DEV, dim=256, theta=10000.0, max_positions=8192)
    j = torch.arange(128, dtype=D)
    ang = 8191.0 * 10000.0 ** (-2.0 * j / 256)
    assert (rope.cos[8191].double().cpu() - torch.cos(ang)).abs().max() < 1e-7      # 64-bit angles, rounded once
    # the same angles taken in 32-bit, as the reference does (llama3.rs:5367-5378), are off by up to 5e-4 here
    ang32 = (torch.tensor(8191.0) * (1.0 / torch.tensor(10000.0).pow(2.0 * torch.arange(128.0) / 256))).double()
    assert (torch.cos(ang32) - torch.cos(ang)).abs().max() < 1e-3
    with pytest.raises(ValueError, match="rotated width"):
        POSITIONS.get("rope")(p, DEV, dim=16, theta=1e4, max_positions=8, rotary_dim=18)


def test_block_part_with_toy_parts_and_an_unfused_norm():
    """The block arrangement alone: toy mixer/feed-forward that scale their input, a norm the stream cannot
    fuse (no `fused` method), and the pre-norm-only form."""
    p = Precision.of("float32")

    class Scale:
        def __init__(self, f): self.f = f
        def forward(self, x, ctx, cache=None): return (x.float() * self.f).contiguous()

    class PlainLayerNorm:                       # no fused(): the stream runs it through forward()
        def forward(self, x, out_dtype, rows=None):
            x = x if rows is None else x.index_select(0, rows.long())
            return torch.nn.functional.layer_norm(x, x.shape[-1:]).to(out_dtype)

    ln = PlainLayerNorm()
    x0 = rnd(7, 40, seed=33, scale=2.0)
    blk = BLOCKS.get("sandwich")(Scale(0.5), Scale(-0.25), {"pre_mixer": ln, "post_mixer": ln, "pre_ff": ln, "post_ff": None})
    s = ResidualStream(x0.clone(), p)
    blk.forward(s, None, None)
    s.flush()
    LN = lambda t: torch.nn.functional.layer_norm(t, t.shape[-1:])
    x1 = x0 + LN(0.5 * LN(x0))
    x2 = x1 - 0.25 * LN(x1)
    assert (s.x - x2).abs().max() < 1e-5
    pre = BLOCKS.get("prenorm")(Scale(2.0), Scale(1.0), {})          # no norms at all: x + 2x, then + that
    s = ResidualStream(x0.clone(), p)
    pre.forward(s, None, None)
    s.flush()
    assert (s.x - 6.0 * x0).abs().max() < 1e-4
