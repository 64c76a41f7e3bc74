"""Each kernel alone against a plain 64-bit reference of the same operation, at sizes other than the
engine's, with inputs made so that a fault shows (a far key among hundreds, a window's edge, scattered
pages)."""
import math

import pytest
import torch
import torch.nn.functional as F

from alice_llm_amd.hip import ops
from plain import gemma2_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"
D = torch.float64
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def close(got, ref, atol, rtol=0.0):
    err = (got.double().cpu() - ref.double().cpu()).abs()
    bound = atol + rtol * ref.double().cpu().abs()
    assert (err <= bound).all(), f"max err {err.max().item():.3e} (bound {bound.min().item():.1e}..)"


# ------------------------------------------------------------------ embedding
@pytest.mark.parametrize("wdt", ["float32", "bfloat16"])
def test_embed(wdt):
    V, H = 301, 72
    table = rnd(V, H, seed=1, dtype=DT[wdt])
    tok = torch.tensor([0, 300, 5, 5, 17], dtype=torch.int32, device=DEV)
    out = torch.empty(5, H, device=DEV)
    ops.embed(tok, table, out, 3.25, V, H)
    close(out, table.double()[tok.long()] * 3.25, 1e-6)


# ------------------------------------------------------------------ residual add and norms
@pytest.mark.parametrize("wdt,odt,full", [("float32", "float32", True), ("bfloat16", "bfloat16", False), ("bfloat16", "float32", True)])
@pytest.mark.parametrize("H", [70, 400, 2304, 5000, 9000])      # 1, 2, 4 and 8 elements a thread; wider than registers hold
def test_add_norm_all_forms(wdt, odt, full, H):
    T = 5
    x0 = rnd(T, H, seed=2, scale=3.0)
    br = rnd(3, T, H, seed=3, scale=0.5)
    wp, wq = rnd(H, seed=4, scale=0.1, dtype=DT[wdt]), rnd(H, seed=5, scale=0.1, dtype=DT[wdt])
    tol = 2e-6 if odt == "float32" else 2 ** -8
    # pre norm only
    out = torch.empty(T, H, dtype=DT[odt], device=DEV)
    x = x0.clone()
    ops.add_norm(x, None, None, wq, out, eps_pre=1e-5, off_pre=1.0, full_precision=full)
    close(out, P.rms_norm(x0.double(), wq.double(), 1e-5), tol, tol)
    assert torch.equal(x, x0)
    # add of a post-normed sum of partials, then pre norm: one kernel
    x = x0.clone()
    ops.add_norm(x, br, wp, wq, out, eps_post=1e-6, eps_pre=1e-5, off_post=1.0, off_pre=0.0, n_partials=3, full_precision=full)
    xr = x0.double() + P.rms_norm(br.double().sum(0), wp.double(), 1e-6)
    close(x, xr, 1e-5)
    close(out, P.rms_norm(xr, wq.double() - 1.0, 1e-5), tol * 4, tol)
    # plain add (no post norm), no output
    x = x0.clone()
    ops.add_norm(x, br[0].contiguous(), None, None, None, full_precision=full)
    close(x, x0.double() + br[0].double(), 1e-6)
    # gathered rows
    rows = torch.tensor([4, 0, 4], dtype=torch.int32, device=DEV)
    out3 = torch.empty(3, H, dtype=DT[odt], device=DEV)
    ops.add_norm(x0.clone(), None, None, wq, out3, eps_pre=1e-5, off_pre=1.0, rows=rows, full_precision=full)
    close(out3, P.rms_norm(x0.double()[rows.long()], wq.double(), 1e-5), tol, tol)


@pytest.mark.parametrize("H", [256, 1000, 2304, 4096, 4608, 5000, 8192])
@pytest.mark.parametrize("S", [1, 3])
@pytest.mark.parametrize("odt", ["float32", "bfloat16"])
def test_add_norm_many_rows(H, S, odt):
    # long prompts take another kernel (a wave per row, two waves from 4,097 elements on) than single tokens do;
    # the last block has a row too few
    T = 333
    x0 = rnd(T, H, seed=2, scale=3.0)
    br = rnd(S, T, H, seed=3, scale=0.5) if S > 1 else rnd(T, H, seed=3, scale=0.5)
    wp, wq = rnd(H, seed=4, scale=0.1, dtype=torch.bfloat16), rnd(H, seed=5, scale=0.1, dtype=torch.bfloat16)
    tol = 2e-6 if odt == "float32" else 2 ** -8
    x = x0.clone()
    out = torch.full((T, H), float("nan"), dtype=DT[odt], device=DEV)
    ops.add_norm(x, br, wp, wq, out, eps_post=1e-6, eps_pre=1e-5, off_post=1.0, off_pre=1.0, n_partials=S, full_precision=False)
    b = br.double().sum(0) if S > 1 else br.double()
    xr = x0.double() + P.rms_norm(b, wp.double(), 1e-6)
    close(x, xr, 1e-5)
    close(out, P.rms_norm(xr, wq.double(), 1e-5), tol * 4, tol)
    # the single-token kernel on the same rows: equal up to the order of the sums
    x2, out2 = x0[:7].clone(), torch.empty(7, H, dtype=DT[odt], device=DEV)
    ops.add_norm(x2, br[:, :7].contiguous() if S > 1 else br[:7].contiguous(), wp, wq, out2, eps_post=1e-6, eps_pre=1e-5,
                 off_post=1.0, off_pre=1.0, n_partials=S, full_precision=False)
    close(x[:7], x2, 2e-6, 1e-6)
    # add only, and norm only
    x = x0.clone()
    ops.add_norm(x, br, None, None, None, n_partials=S, full_precision=False)
    close(x, x0.double() + b, 1e-5)
    ops.add_norm(x0, None, None, wq, out, eps_pre=1e-5, off_pre=0.0, full_precision=False)
    close(out, P.rms_norm(x0.double(), wq.double() - 1.0, 1e-5), tol * 4, tol)
    if H % 32 == 0 and odt == "bfloat16":
        flat = torch.empty((-(-T // 16) * 16) * H, dtype=torch.bfloat16, device=DEV)
        ops.add_norm(x0, None, None, wq, flat, eps_pre=1e-5, off_pre=0.0, full_precision=False, out_layout=ops.LAYOUT_FRAG16)
        assert torch.equal(acts_from_fragments(flat, T, H), out.cpu())


def test_rms_norm_reference_vector_on_device():
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=DEV)                       # llama3.rs:20482-20498
    out = torch.empty_like(x)
    ops.add_norm(x, None, None, torch.zeros(4, device=DEV), out, eps_pre=1e-5, off_pre=1.0, full_precision=True)
    close(out, x.double() / math.sqrt(7.5 + 1e-5), 1e-6)


def test_softcap():
    x = torch.tensor([-1e4, -50.0, -1.0, 0.0, 1e-3, 1.0, 29.0, 300.0, 1e30], device=DEV)
    for full in (True, False):
        y = x.clone()
        ops.softcap_(y, 30.0, full)
        close(y, 30.0 * torch.tanh(x.double() / 30.0), 1e-5 if full else 2e-4)


# ------------------------------------------------------------------ matrix product
LINEAR_SHAPES = [(1, 96, 64), (7, 200, 144), (8, 70, 37), (3, 63, 64), (64, 130, 320), (65, 64, 33), (300, 97, 100)]


@pytest.mark.parametrize("M,N,K", LINEAR_SHAPES)
@pytest.mark.parametrize("xdt,wdt,ydt", [("float32", "float32", "float32"), ("float32", "bfloat16", "float32"),
                                          ("bfloat16", "bfloat16", "bfloat16"), ("bfloat16", "float32", "float32")])
def test_linear_generic(M, N, K, xdt, wdt, ydt):
    x, w = rnd(M, K, seed=6, dtype=DT[xdt]), rnd(N, K, seed=7, scale=0.1, dtype=DT[wdt])
    y = torch.empty(M, N, dtype=DT[ydt], device=DEV)
    full = xdt == "float32"
    ops.linear(x, w, y, n_out=N, k_in=K, full_precision=full, variant=ops.LINEAR_GENERIC)
    ref = x.double() @ w.double().T
    close(y, ref, 1e-5 if ydt == "float32" else 1e-2, 0 if ydt == "float32" else 2 ** -8)
    # softcap epilogue
    y2 = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops.linear(x, w, y2, n_out=N, k_in=K, epilogue=ops.EPI_SOFTCAP, epi_param=2.0, full_precision=full, variant=ops.LINEAR_GENERIC)
    close(y2, 2.0 * torch.tanh(ref / 2.0), 1e-5 if full else 5e-4)


@pytest.mark.parametrize("M,N,K", [(3, 48, 64), (70, 160, 96), (9, 33, 40), (8, 128, 70), (1, 320, 96)])
@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_linear_generic_geglu(M, N, K, dt):
    x, w = rnd(M, K, seed=8, dtype=DT[dt]), rnd(2 * N, K, seed=9, scale=0.3, dtype=DT[dt])
    y = torch.empty(M, N, dtype=DT[dt], device=DEV)
    ops.linear(x, w, y, n_out=N, k_in=K, epilogue=ops.EPI_GEGLU, full_precision=dt == "float32", variant=ops.LINEAR_GENERIC)
    g, u = x.double() @ w.double()[:N].T, x.double() @ w.double()[N:].T
    # values reach about 20: the bound has an absolute part for the sums and a relative part for the product
    close(y, F.gelu(g, approximate="tanh") * u, 2e-5 if dt == "float32" else 2e-2, 1e-5 if dt == "float32" else 2 ** -7)


# ------------------------------------------------------------------ rotation and cache write
def paged(T_max, nKV, d, dtype, n_seq, seed, page=64):
    """Pools with more pages than needed and a scattered block table."""
    per = -(-T_max // page)
    n_pages = per * n_seq + 3
    g = torch.Generator().manual_seed(seed)
    perm = (torch.randperm(n_pages - 1, generator=g) + 1)[:per * n_seq].view(n_seq, per)
    k = torch.zeros(n_pages, nKV, page, d, dtype=dtype, device=DEV)
    return k, torch.zeros_like(k), perm.to(torch.int32).to(DEV)


def fill_pools(kp, vp, bt, k, v, seq, start=0):
    """k, v: [T, nKV, d] of sequence `seq`, written at positions start.."""
    page = kp.shape[2]
    for t in range(k.shape[0]):
        p = int(bt[seq, (start + t) // page])
        kp[p, :, (start + t) % page] = k[t].to(kp.dtype)
        vp[p, :, (start + t) % page] = v[t].to(vp.dtype)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("nH,nKV,d,R", [(4, 1, 16, 16), (6, 3, 24, 24), (2, 2, 40, 16), (3, 1, 256, 256)])
@pytest.mark.parametrize("many", [False, True])      # few tokens and many take different kernels
def test_rope_cache_write(dt, nH, nKV, d, R, many):
    lens, starts = ([5, 270, 1], [0, 60, 130]) if many else ([5, 70, 1], [0, 60, 130])
    T = sum(lens)
    qkv = rnd(T, (nH + 2 * nKV) * d + 8, seed=10, dtype=DT[dt])[:, :].contiguous()       # rows longer than the heads
    pos = torch.tensor([s + i for s, n in zip(starts, lens) for i in range(n)], dtype=torch.int32, device=DEV)
    seq = torch.tensor([b for b, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    kp, vp, bt = paged(384, nKV, d, DT[dt], 3, seed=11)
    theta = 5e5
    j = torch.arange(R // 2, dtype=D)
    ang = torch.arange(400, dtype=D)[:, None] * theta ** (-2.0 * j / R)
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    q_out = torch.empty(T, nH * d, dtype=DT[dt], device=DEV)
    ops.rope_cache_write(qkv, q_out, kp, vp, cos, sin, pos, seq, bt, num_heads=nH, num_kv_heads=nKV, head_dim=d,
                         rotary_dim=R, max_position=int(pos.max()))
    x = qkv.double().cpu()
    q = x[:, :nH * d].view(T, nH, d)
    k = x[:, nH * d:(nH + nKV) * d].view(T, nKV, d)
    v = x[:, (nH + nKV) * d:(nH + 2 * nKV) * d].view(T, nKV, d)
    def rot(a):
        r = P.rope_half_split(a[..., :R], pos.cpu(), theta)
        return torch.cat([r, a[..., R:]], dim=-1)
    tol = 2e-6 if dt == "float32" else 2 ** -7
    close(q_out.view(T, nH, d), rot(q), tol * 4, tol)
    for t in range(T):
        page, off = int(bt[int(seq[t]), int(pos[t]) // 64]), int(pos[t]) % 64
        close(kp[page, :, off], rot(k)[t], tol * 4, tol)
        close(vp[page, :, off], v[t], 0)
    assert float(kp[0].abs().sum()) == 0 and int((kp.abs().sum(dim=(1, 3)) > 0).sum()) == T   # nothing else was touched
    # q only, no cache
    q2 = torch.empty_like(q_out)
    ops.rope_cache_write(qkv, q2, None, None, cos, sin, pos, None, None, num_heads=nH, num_kv_heads=nKV, head_dim=d,
                         rotary_dim=R, max_position=int(pos.max()))
    assert torch.equal(q2, q_out)
    with pytest.raises(ops.HipLibraryError, match="beyond the rotation tables"):
        ops.rope_cache_write(qkv, q2, None, None, cos[:100], sin[:100], pos, None, None, num_heads=nH,
                             num_kv_heads=nKV, head_dim=d, rotary_dim=R, max_position=int(pos.max()))


# ------------------------------------------------------------------ attention
def attention_case(dt, nH, nKV, d, lens, new, cap, window, seed, crafted=None):
    """Sequences of total lengths `lens`, whose last `new[i]` tokens are the step's queries."""
    B = len(lens)
    kp, vp, bt = paged(max(lens), nKV, d, DT[dt], B, seed)
    qs, refs, pos, seq = [], [], [], []
    scale = 1.0 / math.sqrt(d * 1.7)
    for b, (L, n) in enumerate(zip(lens, new)):
        g = torch.Generator().manual_seed(seed * 100 + b)
        q = torch.randn(L, nH, d, generator=g, dtype=D)
        k = torch.randn(L, nKV, d, generator=g, dtype=D)
        v = torch.randn(L, nKV, d, generator=g, dtype=D)
        if crafted is not None:
            crafted(b, q, k, v)
        q, k, v = (t.to(DT[dt]).double() for t in (q, k, v))
        fill_pools(kp, vp, bt, k, v, b)
        refs.append(P.attention_core(q, k, v, scale, cap, window)[L - n:])
        qs.append(q[L - n:])
        pos += list(range(L - n, L))
        seq += [b] * n
    q = torch.cat(qs).reshape(-1, nH * d).to(DT[dt]).to(DEV)
    return q, kp, vp, bt, torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(seq, dtype=torch.int32, device=DEV), \
        torch.cat(refs).reshape(-1, nH * d), scale


ATT_SHAPES = [(4, 1, 16), (6, 3, 24), (8, 4, 64), (2, 1, 256), (5, 5, 40)]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("nH,nKV,d", ATT_SHAPES)
@pytest.mark.parametrize("cap,window", [(None, None), (5.0, 50), (50.0, 7)])
def test_attention_generic_prompts_and_decode(dt, nH, nKV, d, cap, window):
    for lens, new in (((5, 130, 66), (5, 130, 66)), ((200, 1, 77), (1, 1, 1)), ((150, 64), (20, 3))):
        q, kp, vp, bt, pos, seq, ref, scale = attention_case(dt, nH, nKV, d, lens, new, cap, window, seed=3)
        out = torch.empty_like(q)
        ops.attention_generic(q, kp, vp, out, pos, seq, bt, num_heads=nH, scale=scale, softcap=cap, window=window,
                              max_position=max(lens) - 1, full_precision=dt == "float32")
        close(out, ref, 2e-5 if dt == "float32" else 2e-2)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_attention_far_key_and_window_edge(dt):
    nH, nKV, d, L = 4, 2, 32, 700
    # one far key (position 3) whose score towers over hundreds of others: the output is its value
    def far(b, q, k, v):
        k[3] = 0; k[3, :, 0] = 40.0
        q[L - 1] = 0; q[L - 1, :, 0] = 40.0
    q, kp, vp, bt, pos, seq, ref, scale = attention_case(dt, nH, nKV, d, (L,), (1,), None, None, seed=4, crafted=far)
    out = torch.empty_like(q)
    kw = dict(num_heads=nH, scale=scale, max_position=L - 1, full_precision=dt == "float32")
    ops.attention_generic(q, kp, vp, out, pos, seq, bt, softcap=None, window=None, **kw)
    close(out, ref, 2e-5 if dt == "float32" else 2e-2)
    v3 = vp[int(bt[0, 0]), :, 3].double().cpu()
    assert (out.view(nH, d)[0].double().cpu() - v3[0]).abs().max() < 1e-2
    # a window of 100: the towering key at the first position outside (L - 101) is not seen, the one at the
    # first position inside (L - 100) wins
    for where, seen in ((L - 101, False), (L - 100, True)):
        def edge(b, q, k, v, where=where):
            k[where] = 0; k[where, :, 0] = 40.0; v[where] = 7.0
            q[L - 1] = 0; q[L - 1, :, 0] = 40.0
        q, kp, vp, bt, pos, seq, ref, scale = attention_case(dt, nH, nKV, d, (L,), (1,), None, 100, seed=5, crafted=edge)
        out = torch.empty_like(q)
        ops.attention_generic(q, kp, vp, out, pos, seq, bt, softcap=None, window=100, **kw)
        close(out, ref, 2e-5 if dt == "float32" else 2e-2)
        assert (abs(float(out[0, 0]) - 7.0) < 1e-2) == seen


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("cap,window", [(None, None), (5.0, 40)])
def test_attention_generic_with_a_distance_bias_at_the_score_stage(dt, cap, window):
    """A position term at the score stage as a parameter of the kernel: head h's capped score of key k for the
    query at position p gets slope[h] * (k - p) added.  Against a dense reference written here (the plain
    implementation of the product's architecture has no such term): prompts on a cached prefix and single tokens.
    Slopes of zero give the bits of the call without slopes, and a steep slope leaves every query its own value."""
    nH, nKV, d = 6, 2, 24
    slopes = torch.tensor([0.0, 0.5, 0.25, 0.125, 0.0625, 0.03125], dtype=D)
    for lens, new in (((70, 131), (70, 9)), ((150, 3, 65), (1, 1, 1))):
        B = len(lens)
        kp, vp, bt = paged(max(lens), nKV, d, DT[dt], B, 8)
        scale = 1.0 / math.sqrt(d)
        qs, refs, pos, seq = [], [], [], []
        for b, (L, n) in enumerate(zip(lens, new)):
            g = torch.Generator().manual_seed(800 + b)
            q, k, v = (torch.randn(L, h, d, generator=g, dtype=D).to(DT[dt]).double() for h in (nH, nKV, nKV))
            fill_pools(kp, vp, bt, k, v, b)
            ar = torch.arange(L)
            dist = (ar[None, :] - ar[:, None]).double()                         # key position - query position
            out = torch.empty(L, nH, d, dtype=D)
            for h in range(nH):
                sc = (q[:, h] @ k[:, h // (nH // nKV)].T) * scale
                if cap is not None:
                    sc = cap * torch.tanh(sc / cap)
                sc = sc + slopes[h] * dist
                seen = (dist <= 0) & ((dist > -window) if window else torch.ones_like(dist, dtype=torch.bool))
                out[:, h] = torch.softmax(sc.masked_fill(~seen, float("-inf")), dim=-1) @ v[:, h // (nH // nKV)]
            refs.append(out[L - n:])
            qs.append(q[L - n:])
            pos += list(range(L - n, L))
            seq += [b] * n
        q = torch.cat(qs).reshape(-1, nH * d).to(DT[dt]).to(DEV)
        pos_t, seq_t = (torch.tensor(a, dtype=torch.int32, device=DEV) for a in (pos, seq))
        ref = torch.cat(refs).reshape(-1, nH * d)
        kw = dict(num_heads=nH, scale=scale, softcap=cap, window=window, max_position=max(lens) - 1, full_precision=dt == "float32")
        out = torch.empty_like(q)
        ops.attention_generic(q, kp, vp, out, pos_t, seq_t, bt, bias_slopes=slopes.float().to(DEV), **kw)
        close(out, ref, 2e-5 if dt == "float32" else 2e-2)
        plain, zero = torch.empty_like(q), torch.empty_like(q)
        ops.attention_generic(q, kp, vp, plain, pos_t, seq_t, bt, **kw)
        ops.attention_generic(q, kp, vp, zero, pos_t, seq_t, bt, bias_slopes=torch.zeros(nH, device=DEV), **kw)
        assert torch.equal(plain, zero) and (plain.float() - out.float()).abs().max() > 0.05
        steep = torch.empty_like(q)
        ops.attention_generic(q, kp, vp, steep, pos_t, seq_t, bt, bias_slopes=torch.full((nH,), 200.0, device=DEV), **kw)
        own = torch.stack([vp[int(bt[b, p // 64]), :, p % 64] for b, p in zip(seq, pos)]).float()          # [T, nKV, d]
        assert (steep.view(-1, nKV, nH // nKV, d).float() - own[:, :, None]).abs().max() < 1e-5
    with pytest.raises(ops.HipLibraryError, match="bias_slopes"):
        ops.attention_generic(q, kp, vp, out, pos_t, seq_t, bt, bias_slopes=torch.zeros(nH + 1, device=DEV), **kw)


def test_attention_refuses_sizes_it_does_not_cover():
    q, kp, vp, bt, pos, seq, ref, scale = attention_case("float32", 2, 1, 16, (9,), (9,), None, None, seed=6)
    out = torch.empty_like(q)
    with pytest.raises(ops.HipLibraryError, match="beyond the block table"):
        ops.attention_generic(q, kp, vp, out, pos, seq, bt, num_heads=2, scale=scale, softcap=None, window=None,
                              max_position=64, full_precision=True)
    with pytest.raises(ops.HipLibraryError, match="head counts"):
        ops.attention_generic(torch.empty(9, 48, device=DEV), kp.repeat(1, 2, 1, 1), vp.repeat(1, 2, 1, 1),
                              torch.empty(9, 48, device=DEV), pos, seq, bt, num_heads=3, scale=scale, softcap=None,
                              window=None, max_position=8, full_precision=True)
    big = torch.zeros(2, 1, 64, 272, device=DEV)
    with pytest.raises(ops.HipLibraryError, match="head_dim 272"):
        ops.attention_generic(torch.empty(9, 272, device=DEV), big, big, torch.empty(9, 272, device=DEV), pos, seq, bt,
                              num_heads=1, scale=scale, softcap=None, window=None, max_position=8, full_precision=True)


# ------------------------------------------------------------------ sampling
def test_argmax_lowest_index_on_ties():
    x = rnd(5, 1000, seed=12)
    x[1, 7] = x[1, 900] = 50.0
    x[2] = 0.0
    x[3, 999] = 60.0
    got = ops.argmax(x).cpu().tolist()
    assert got == [int(x[0].argmax()), 7, 0, 999, int(x[4].argmax())]
    assert ops.argmax(torch.tensor([[0.7, 0.5, 0.7, 0.3]], device=DEV)).item() == 0    # llama3.rs:21263-21269


def test_sample_reference_vectors():
    probs = torch.tensor([[0.1, 0.2, 0.7]] * 3 + [[0.5, 0.5, 0.0]] * 3, device=DEV)     # integration_tests.rs
    u = torch.tensor([0.05, 0.25, 0.95, 0.0, 0.49, 0.51], device=DEV)
    assert ops.sample(probs.log(), u, 1.0).cpu().tolist() == [0, 1, 2, 0, 0, 1]
    only = torch.tensor([[0.0, 0.0, 1.0, 0.0]], device=DEV).log()                        # llama3.rs:21390-21399
    assert all(ops.sample(only, torch.tensor([x], device=DEV), 1.0).item() == 2 for x in (0.0, 0.5, 0.999999))


@pytest.mark.parametrize("V", [384, 5000, 256000])
def test_sample_matches_plain(V):
    B = 6
    logits = rnd(B, V, seed=13, scale=3.0)
    g = torch.Generator().manual_seed(14)
    for temperature, top_k, top_p in ((0.8, 0, 1.0), (1.5, 40, 1.0), (0.7, 0, 0.9), (1.0, 50, 0.5), (1e-3, 0, 1.0)):
        u = torch.rand(B, generator=g)
        check_samples(logits, u, temperature, top_k, top_p)


def top_p_ties_kept(x, p):
    """plain_top_p, and every value tied with the last kept one as well: what the kernel's threshold keeps."""
    kept = P.plain_top_p(x, p)
    return torch.where(x >= kept[kept > -math.inf].min(), x, torch.full_like(x, -math.inf))


def check_samples(logits, u, temperature, top_k, top_p):
    got = ops.sample(logits, u.to(DEV), temperature, top_k, top_p).cpu().tolist()
    for b in range(logits.shape[0]):
        x = top_p_ties_kept(P.plain_top_k(logits[b].double().cpu() / temperature, top_k), top_p)
        probs = P.plain_softmax(x)
        want = P.plain_inverse_cdf(probs, float(u[b]))
        if got[b] != want:
            # a draw within rounding of a boundary of the cumulative sum may fall on either side
            cdf = torch.cumsum(probs, 0)
            assert x[got[b]] > -math.inf and abs(float(cdf[min(got[b], want)]) - float(u[b])) < 1e-5, (b, got[b], want)
    return got


@pytest.mark.parametrize("V", [383, 5000, 70002])
def test_sample_where_the_kept_set_is_large_or_tied(V):
    """Rows whose kept set does not fit the kernel's short list, and ties at both thresholds."""
    g = torch.Generator().manual_seed(16)
    B = 5
    flat = torch.zeros(B, V)                                          # every token tied
    steps = torch.randint(0, 3, (B, V), generator=g).float()          # three values, thousands of ties each
    peaks = rnd(B, V, seed=17, scale=0.1).cpu()
    peaks[:, 11] = peaks[:, V - 2] = 9.0                              # two tied peaks far above a flat rest
    holes = rnd(B, V, seed=18, scale=3.0).cpu()
    holes[:, ::3] = -math.inf                                         # masked tokens are never drawn
    wide = rnd(B, V, seed=19, scale=0.5).cpu()                        # a nucleus of most of the vocabulary
    broad = rnd(B, V, seed=23, scale=2.0).cpu()                       # a kept set of some thousands: the list in memory
    for logits in (flat, steps, peaks, holes, wide, broad):
        logits = logits.to(DEV)
        for temperature, top_k, top_p in ((1.0, 0, 0.9), (1.0, 7, 1.0), (0.9, V - 1, 0.95), (1.3, 6000, 0.999),
                                          (1.0, 2, 0.6), (0.5, 0, 0.3)):
            u = torch.rand(B, generator=g)
            got = check_samples(logits, u, temperature, top_k, top_p)
            assert all(logits[b, t] > -math.inf for b, t in enumerate(got))
    u = torch.tensor([0.1, 0.3, 0.5, 0.7, 0.9])
    assert set(ops.sample(peaks.to(DEV), u.to(DEV), 1.0, 2, 1.0).cpu().tolist()) == {11, V - 2}
    assert set(ops.sample(peaks.to(DEV), u.to(DEV), 1.0, 1, 1.0).cpu().tolist()) == {11, V - 2}   # ties are kept


def test_sample_depends_on_the_row_alone():
    """The same row gives the same token wherever it stands in the batch, whatever the other rows hold."""
    V = 70002
    row = rnd(1, V, seed=20, scale=2.0)
    other = rnd(7, V, seed=21, scale=5.0)
    g = torch.Generator().manual_seed(22)
    for temperature, top_k, top_p in ((1.0, 0, 1.0), (0.8, 40, 0.9), (1.2, 0, 0.95), (1.0, 30000, 0.9)):
        for _ in range(4):
            u = float(torch.rand(1, generator=g))
            alone = ops.sample(row, torch.tensor([u], device=DEV), temperature, top_k, top_p).item()
            for place in (0, 3, 7):
                batch = torch.cat([other[:place], row, other[place:]])
                us = torch.rand(8, generator=g)
                us[place] = u
                assert ops.sample(batch, us.to(DEV), temperature, top_k, top_p)[place].item() == alone


def test_sample_frequencies():
    logits = torch.tensor([[0.0, 0.0]], device=DEV).repeat(4000, 1)                       # llama3.rs:21401-21413
    u = torch.rand(4000, generator=torch.Generator().manual_seed(15)).to(DEV)
    ones = int(ops.sample(logits, u, 1.0).sum())
    assert abs(ones - 2000) < 150
    skew = torch.tensor([[0.0, 1.0, 2.0, 3.0]], device=DEV).repeat(4000, 1)
    cold = ops.sample(skew, u, 0.01)
    hot = ops.sample(skew, u, 1000.0)
    assert int((cold == 3).sum()) == 4000 and 800 < int((hot == 0).sum()) < 1200          # llama3.rs:21339-21363
    topk = ops.sample(skew, u, 1000.0, 2, 1.0)
    assert set(topk.cpu().tolist()) == {2, 3}


# ------------------------------------------------------------------ matrix-core matrix products
def frag_reference(w):
    """The fragment layout written out in plain indexing: [N/16][K/32][lane = g*16 + r][8]."""
    N, K = w.shape
    Np, Kp = -(-N // 16) * 16, -(-K // 32) * 32
    wp = torch.zeros(Np, Kp, dtype=w.dtype)
    wp[:N, :K] = w.cpu()
    return wp.view(Np // 16, 16, Kp // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(-1)


def test_fragment_layout():
    for N, K in ((16, 32), (40, 72), (96, 64), (33, 8)):
        w = rnd(N, K, seed=N, dtype=torch.bfloat16)
        assert torch.equal(ops.to_frag16(w).cpu(), frag_reference(w))
    assert ops.fragment_layout_supported(96, 64, ops.EPI_NONE) and not ops.fragment_layout_supported(96, 36, ops.EPI_NONE)
    assert ops.fragment_layout_supported(64, 64, ops.EPI_GEGLU) and not ops.fragment_layout_supported(48, 64, ops.EPI_GEGLU)


MFMA_SHAPES = [(1, 96, 64), (7, 208, 144), (16, 4096, 256), (17, 130, 320), (33, 64, 96), (64, 2304, 1024),
               (65, 304, 160), (128, 256, 64), (300, 1000, 416), (1000, 80, 2048)]


@pytest.mark.parametrize("M,N,K", MFMA_SHAPES)
@pytest.mark.parametrize("ydt", ["float32", "bfloat16"])
def test_linear_mfma(M, N, K, ydt):
    x, w = rnd(M, K, seed=16, dtype=torch.bfloat16), rnd(N, K, seed=17, scale=0.1, dtype=torch.bfloat16)
    wf = ops.to_frag16(w)
    ref = x.double() @ w.double().T
    atol, rtol = (2e-4, 1e-5) if ydt == "float32" else (1e-2, 2 ** -8)
    variants = [ops.LINEAR_MFMA] + ([ops.LINEAR_SKINNY] if M <= 64 else [])
    for variant in variants:
        y = torch.full((M, N), float("nan"), dtype=DT[ydt], device=DEV)
        ops.linear(x, wf, y, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, variant=variant, full_precision=False)
        close(y, ref, atol * math.sqrt(K / 64), rtol)
        y2 = torch.empty(M, N, dtype=torch.float32, device=DEV)
        ops.linear(x, wf, y2, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, epilogue=ops.EPI_SOFTCAP, epi_param=3.0,
                   variant=variant, full_precision=False)
        close(y2, 3.0 * torch.tanh(ref / 3.0), 1e-3)
    if M <= 64:
        for split in (2, 3, 8):
            yp = torch.full((split, M, N), float("nan"), dtype=torch.float32, device=DEV)
            ops.linear(x, wf, yp, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, split_k=split, variant=ops.LINEAR_SKINNY,
                       full_precision=False)
            close(yp.sum(0), ref, 2e-4 * math.sqrt(K / 64), 1e-5)


@pytest.mark.parametrize("M", [3, 20, 40, 64])
def test_linear_streaming_with_six_row_tiles(M):
    """Shapes for which the streaming kernel takes six row tiles a block (the cost rule of the launcher picks them
    where three blocks' worth of tiles would otherwise wait for one another), with tile counts that six does not
    divide: gate/up of 577 pairs, and a product of 145 row tiles in slices of the inner dimension."""
    K = 512
    x = rnd(M, K, seed=80, dtype=torch.bfloat16)
    w2 = rnd(2 * 9232, K, seed=81, scale=0.3, dtype=torch.bfloat16)
    gate, up = x.double() @ w2.double()[:9232].T, x.double() @ w2.double()[9232:].T
    yg = torch.full((M, 9232), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear(x, ops.to_frag16(w2), yg, n_out=9232, k_in=K, layout=ops.LAYOUT_FRAG16, epilogue=ops.EPI_GEGLU, full_precision=False)
    close(yg, F.gelu(gate, approximate="tanh") * up, 2e-2, 2 ** -7)
    N, K = 2320, 9216
    x, w = rnd(M, K, seed=82, dtype=torch.bfloat16), rnd(N, K, seed=83, scale=0.1, dtype=torch.bfloat16)
    split = ops.linear_split_hint(M, N, K, ops.LAYOUT_FRAG16)
    assert split > 1
    yp = torch.full((split, M, N), float("nan"), dtype=torch.float32, device=DEV)
    ops.linear(x, ops.to_frag16(w), yp, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, split_k=split, variant=ops.LINEAR_SKINNY,
               full_precision=False)
    close(yp.sum(0), x.double() @ w.double().T, 2e-4 * math.sqrt(K / 64), 1e-5)


def test_between_33_and_64_tokens_the_rule_picks_a_kernel_and_both_agree():
    """From 33 to 64 tokens with activations in fragment order the launcher takes the tiled kernel's narrow tiles where
    their blocks come close to one a CU, the streaming kernel elsewhere; whichever it takes, the sums are those of
    the streaming kernel up to rounding, and the number of slices it proposes is one it can run."""
    for M, N, K in ((40, 2304, 9216), (64, 2304, 2048), (64, 4096, 2304), (33, 8192, 512), (50, 1024, 8192)):
        x, w = rnd(M, K, seed=95, dtype=torch.bfloat16), rnd(N, K, seed=96, scale=0.1, dtype=torch.bfloat16)
        wf, xf = ops.to_frag16(w), acts_to_fragments(x)
        split = ops.linear_split_hint(M, N, K, ops.LAYOUT_FRAG16)
        shape = (split, M, N) if split > 1 else (M, N)
        a = torch.full(shape, float("nan"), dtype=torch.float32, device=DEV)
        b = torch.full(shape, float("nan"), dtype=torch.float32, device=DEV)
        ops.linear(xf, wf, a, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, split_k=split, full_precision=False, rows=M,
                   x_layout=ops.LAYOUT_FRAG16)
        ops.linear(xf, wf, b, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, split_k=split, variant=ops.LINEAR_SKINNY,
                   full_precision=False, rows=M, x_layout=ops.LAYOUT_FRAG16)
        ref = x.double() @ w.double().T
        for y in (a, b):
            close(y.sum(0) if split > 1 else y, ref, 2e-4 * math.sqrt(K / 64), 1e-5)


@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (5, 9216, 128), (40, 416, 160), (64, 48, 96), (200, 304, 96), (129, 2048, 64)])
def test_linear_mfma_geglu(M, N, K):
    x, w = rnd(M, K, seed=18, dtype=torch.bfloat16), rnd(2 * N, K, seed=19, scale=0.3, dtype=torch.bfloat16)
    wf = ops.to_frag16(w)
    g, u = x.double() @ w.double()[:N].T, x.double() @ w.double()[N:].T
    ref = F.gelu(g, approximate="tanh") * u
    for variant in [ops.LINEAR_MFMA] + ([ops.LINEAR_SKINNY] if M <= 64 else []):
        y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.linear(x, wf, y, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, epilogue=ops.EPI_GEGLU, variant=variant, full_precision=False)
        close(y, ref, 2e-2, 2 ** -7)


@pytest.mark.parametrize("M", [1, 8, 16, 24])
def test_linear_mfma_matrices_read_with_the_streaming_hint(M):
    """Matrices of 96 MB or more are read by the streaming kernel with the streaming hint (another instantiation of
    the kernel): the same sums as the tiled kernel, which reads them plainly, and as the plain product."""
    N, K = 26000, 2048                                       # 106 MB in bfloat16
    g = torch.Generator(device=DEV).manual_seed(5)
    w = (torch.randn(N, K, generator=g, device=DEV) * 0.1).to(torch.bfloat16)
    x = rnd(M, K, seed=6, dtype=torch.bfloat16)
    wf = ops.to_frag16(w)
    ref = (x.double() @ w.double().T).cpu()
    for epi, param, want in ((ops.EPI_NONE, 0.0, ref), (ops.EPI_SOFTCAP, 3.0, 3.0 * torch.tanh(ref / 3.0))):
        ys = []
        for variant in (ops.LINEAR_SKINNY, ops.LINEAR_MFMA):
            for frag_in in (True, False):
                y = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
                ops.linear(acts_to_fragments(x) if frag_in else x, wf, y, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, epilogue=epi,
                           epi_param=param, variant=variant, full_precision=False, rows=M,
                           x_layout=ops.LAYOUT_FRAG16 if frag_in else ops.LAYOUT_ROW)
                close(y, want, 1e-3, 1e-5)
                ys.append(y)
        assert torch.equal(ys[0], ys[1])                     # with the hint (fragments in) and without (rows in)


def test_linear_mfma_rows_do_not_depend_on_the_batch():
    # a token's output is the same whatever else is in the batch, within each kernel
    x, w = rnd(64, 320, seed=20, dtype=torch.bfloat16), rnd(208, 320, seed=21, scale=0.1, dtype=torch.bfloat16)
    wf = ops.to_frag16(w)
    def run(xx, variant):
        y = torch.empty(xx.shape[0], 208, dtype=torch.float32, device=DEV)
        ops.linear(xx, wf, y, n_out=208, k_in=320, layout=ops.LAYOUT_FRAG16, variant=variant, full_precision=False)
        return y
    for variant in (ops.LINEAR_SKINNY, ops.LINEAR_MFMA):
        full = run(x, variant)
        assert torch.equal(run(x[5:6].contiguous(), variant)[0], full[5])
        assert torch.equal(run(x[:33].contiguous(), variant), full[:33])


def acts_to_fragments(x):
    """Activations [M, K] (K a multiple of 32) in fragment order, written out in plain indexing:
    [M/16][K/32][lane = g*16 + r][8] holds x[16 mt + r][32 kt + 8 g + e]; rows padded with NaN so that a
    kernel that lets a padded row into a real one shows."""
    M, K = x.shape
    Mp = -(-M // 16) * 16
    xp = torch.full((Mp, K), float("nan"), dtype=x.dtype)
    xp[:M] = x.cpu()
    return xp.view(Mp // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(-1).to(DEV)


def acts_from_fragments(flat, M, K):
    Mp = -(-M // 16) * 16
    return flat.cpu().view(Mp // 16, K // 32, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(Mp, K)[:M]


@pytest.mark.parametrize("M,N,K", [(1, 96, 64), (7, 224, 160), (16, 4096, 256), (17, 160, 320), (33, 64, 96), (64, 2304, 1024),
                                   (40, 65536 + 32, 64), (130, 224, 160), (300, 96, 64), (1000, 2304, 96)])
def test_linear_mfma_activations_in_fragment_order(M, N, K):
    x, w = rnd(M, K, seed=16, dtype=torch.bfloat16), rnd(N, K, seed=17, scale=0.1, dtype=torch.bfloat16)
    wf, xf = ops.to_frag16(w), acts_to_fragments(x)
    assert torch.equal(acts_from_fragments(xf, M, K), x.cpu())
    row = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.linear(x, wf, row, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, full_precision=False)
    close(row, x.double() @ w.double().T, 1e-2 * math.sqrt(K / 64), 2 ** -8)
    # reading fragments, writing rows: the same bits as from rows (float32 partial sums too)
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear(xf, wf, y, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, full_precision=False, rows=M, x_layout=ops.LAYOUT_FRAG16)
    assert torch.equal(y, row)
    if N < 65536:
        for split in (1, 2):
            shape = (split, M, N) if split > 1 else (M, N)
            a, b = torch.empty(shape, device=DEV), torch.empty(shape, device=DEV)
            ops.linear(x, wf, a, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, split_k=split, full_precision=False)
            ops.linear(xf, wf, b, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, split_k=split, full_precision=False, rows=M,
                       x_layout=ops.LAYOUT_FRAG16)
            assert torch.equal(a, b)
    # writing fragments
    for src, lay in ((x, ops.LAYOUT_ROW), (xf, ops.LAYOUT_FRAG16)):
        yf = torch.full(((-(-M // 16) * 16) * N,), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.linear(src, wf, yf, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, full_precision=False, rows=M, x_layout=lay,
                   y_layout=ops.LAYOUT_FRAG16)
        assert torch.equal(acts_from_fragments(yf, M, N), row.cpu())


@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (5, 9216, 128), (40, 416, 160), (64, 96, 96), (200, 320, 96), (513, 2048, 64)])
def test_linear_mfma_geglu_in_fragment_order(M, N, K):
    x, w = rnd(M, K, seed=18, dtype=torch.bfloat16), rnd(2 * N, K, seed=19, scale=0.3, dtype=torch.bfloat16)
    wf, xf = ops.to_frag16(w), acts_to_fragments(x)
    row = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.linear(x, wf, row, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, epilogue=ops.EPI_GEGLU, full_precision=False)
    yf = torch.full(((-(-M // 16) * 16) * N,), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear(xf, wf, yf, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, epilogue=ops.EPI_GEGLU, full_precision=False, rows=M,
               x_layout=ops.LAYOUT_FRAG16, y_layout=ops.LAYOUT_FRAG16)
    assert torch.equal(acts_from_fragments(yf, M, N), row.cpu())


@pytest.mark.parametrize("M,N,K", [(65, 48, 64), (100, 304, 160), (128, 2304, 2048), (200, 1000, 416), (257, 80, 1184), (700, 130, 96),
                                   (33, 304, 160), (48, 1000, 416), (64, 2304, 2048)])
def test_linear_tiled_with_narrow_wave_tiles(M, N, K):
    """The tiled kernel's wave tiles of 16 and 32 output features (prompts of a few hundred tokens, and 33 to 64
    tokens where they beat the streaming kernel), forced whatever the cost rule would pick: float32 sums whole and in slices of the inner dimension, and the GeGLU epilogue, with
    token counts that end inside a block, tile counts that a block's four waves do not divide, and inner dimensions
    that are no multiple of a stage."""
    x, w = rnd(M, K, seed=90, dtype=torch.bfloat16), rnd(N, K, seed=91, scale=0.1, dtype=torch.bfloat16)
    wf, xf = ops.to_frag16(w), acts_to_fragments(x)
    ref = x.double() @ w.double().T
    wide = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops.linear(x, wf, wide, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, variant=ops.LINEAR_MFMA, full_precision=False)
    for variant in (ops.LINEAR_TILED_W16, ops.LINEAR_TILED_W32):
        for split in (1, 2, 3):
            if split > 1 and K // 32 < 2 * split:
                continue
            y = torch.full((split, M, N) if split > 1 else (M, N), float("nan"), dtype=torch.float32, device=DEV)
            ops.linear(xf, wf, y, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, split_k=split, variant=variant, full_precision=False,
                       rows=M, x_layout=ops.LAYOUT_FRAG16)
            if split == 1:
                assert torch.equal(y, wide)                  # the same products in the same order
            else:
                close(y.sum(0), ref, 2e-4 * math.sqrt(K / 64), 1e-5)
    if N % 16 == 0:
        w2 = rnd(2 * N, K, seed=92, scale=0.3, dtype=torch.bfloat16)
        gate, up = x.double() @ w2.double()[:N].T, x.double() @ w2.double()[N:].T
        for y_layout in (ops.LAYOUT_ROW,) + ((ops.LAYOUT_FRAG16,) if N % 32 == 0 else ()):
            frag = y_layout == ops.LAYOUT_FRAG16
            yg = torch.full(((-(-M // 16) * 16) * N,) if frag else (M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
            ops.linear(xf, ops.to_frag16(w2), yg, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, epilogue=ops.EPI_GEGLU,
                       variant=ops.LINEAR_TILED_W32, full_precision=False, rows=M, x_layout=ops.LAYOUT_FRAG16, y_layout=y_layout)
            got = acts_from_fragments(yg, M, N).to(DEV) if frag else yg
            close(got, F.gelu(gate, approximate="tanh") * up, 2e-2 * math.sqrt(K / 64), 2 ** -7)
    # what has no narrow kernel says so
    y = torch.empty(M, N, dtype=torch.float32, device=DEV)
    with pytest.raises(ops.HipLibraryError, match="wave tile"):
        ops.linear(x, wf, y, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, variant=ops.LINEAR_TILED_W16, full_precision=False)


def test_tiled_plan_splits_within_the_inner_dimension():
    """The number of slices that the rule proposes for prompts keeps at least 16 k-tiles a slice and is one for
    matrices that fill the chip by themselves."""
    for M in (65, 128, 300, 512, 1024, 2048, 5000):
        for N, K in ((2304, 2048), (2304, 9216), (4608, 36864), (18432, 2304), (64, 96), (3584, 512)):
            s = ops.linear_split_hint(M, N, K, ops.LAYOUT_FRAG16)
            assert 1 <= s <= 8 and (s == 1 or (K // 32) // s >= 16), (M, N, K, s)
    assert ops.linear_split_hint(4096, 18432, 2304, ops.LAYOUT_FRAG16) == 1


def test_linear_refuses_fragment_order_it_cannot_take():
    x, w = rnd(8, 40, seed=1, dtype=torch.bfloat16), rnd(48, 40, seed=2, dtype=torch.bfloat16)
    y = torch.empty(8, 48, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ops.HipLibraryError, match="K % 32"):      # inner width no multiple of 32
        ops.linear(torch.empty(16 * 40, dtype=torch.bfloat16, device=DEV), ops.to_frag16(w), y, n_out=48, k_in=40,
                   layout=ops.LAYOUT_FRAG16, full_precision=False, rows=8, x_layout=ops.LAYOUT_FRAG16)
    w2 = rnd(48, 64, seed=2, dtype=torch.bfloat16)
    with pytest.raises(ops.HipLibraryError, match="fragment order"):    # output width no multiple of 32
        ops.linear(rnd(8, 64, dtype=torch.bfloat16), ops.to_frag16(w2), torch.empty(16 * 48, dtype=torch.bfloat16, device=DEV),
                   n_out=48, k_in=64, layout=ops.LAYOUT_FRAG16, full_precision=False, rows=8, y_layout=ops.LAYOUT_FRAG16)
    with pytest.raises(ops.HipLibraryError, match="generic kernel"):   # the 32-bit path has rows only
        ops.linear(torch.empty(16 * 64, dtype=torch.bfloat16, device=DEV), w2, y, n_out=48, k_in=64, full_precision=True, rows=8,
                   x_layout=ops.LAYOUT_FRAG16)


@pytest.mark.parametrize("T,H", [(1, 64), (8, 2304), (37, 96), (64, 4608), (20, 10016)])
def test_add_norm_writes_fragment_order(T, H):
    x0, br = rnd(T, H, seed=2, scale=3.0), rnd(2, T, H, seed=3, scale=0.5)
    wp, wq = rnd(H, seed=4, scale=0.1, dtype=torch.bfloat16), rnd(H, seed=5, scale=0.1, dtype=torch.bfloat16)
    xa, xb = x0.clone(), x0.clone()
    row = torch.empty(T, H, dtype=torch.bfloat16, device=DEV)
    ops.add_norm(xa, br, wp, wq, row, eps_post=1e-6, eps_pre=1e-5, off_post=1.0, off_pre=1.0, n_partials=2, full_precision=False)
    flat = torch.full(((-(-T // 16) * 16) * H,), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.add_norm(xb, br, wp, wq, flat, eps_post=1e-6, eps_pre=1e-5, off_post=1.0, off_pre=1.0, n_partials=2, full_precision=False,
                 out_layout=ops.LAYOUT_FRAG16)
    assert torch.equal(xa, xb) and torch.equal(acts_from_fragments(flat, T, H), row.cpu())
    # gathered rows (what the output head reads)
    rows = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32, device=DEV)
    row = torch.empty(3, H, dtype=torch.bfloat16, device=DEV)
    ops.add_norm(xa, None, None, wq, row, eps_pre=1e-5, off_pre=1.0, rows=rows, full_precision=False)
    flat = torch.empty(16 * H, dtype=torch.bfloat16, device=DEV)
    ops.add_norm(xa, None, None, wq, flat, eps_pre=1e-5, off_pre=1.0, rows=rows, full_precision=False, out_layout=ops.LAYOUT_FRAG16)
    assert torch.equal(acts_from_fragments(flat, 3, H), row.cpu())


def test_embed_from_fragment_layout():
    V, H = 301, 72
    table = rnd(V, H, seed=1, dtype=torch.bfloat16)
    tok = torch.tensor([0, 300, 5, 5, 17, 16, 15], dtype=torch.int32, device=DEV)
    out = torch.empty(7, H, device=DEV)
    ops.embed(tok, ops.to_frag16(table), out, 3.25, V, H, ops.LAYOUT_FRAG16)
    close(out, table.double()[tok.long()] * 3.25, 1e-6)


# ------------------------------------------------------------------ matrix-core attention over the fragment cache layout
def frag_case(nH, nKV, d, lens, new, cap, window, seed, crafted=None, dense=False):
    """Like attention_case, with the cache filled by rope_cache_write in the fragment layout (no rotation).
    dense: the reference through the plain implementation's masked matrix form on the GPU (long sequences)."""
    B = len(lens)
    kp, vp, bt = paged(max(lens), nKV, d, torch.bfloat16, B, seed)
    qs, refs = [], []
    scale = 1.0 / math.sqrt(d * 1.7)
    for b, (L, n) in enumerate(zip(lens, new)):
        g = torch.Generator().manual_seed(seed * 100 + b)
        q = torch.randn(L, nH, d, generator=g, dtype=D)
        k = torch.randn(L, nKV, d, generator=g, dtype=D)
        v = torch.randn(L, nKV, d, generator=g, dtype=D)
        if crafted is not None:
            crafted(b, q, k, v)
        q, k, v = (t.to(torch.bfloat16) for t in (q, k, v))
        qkv = torch.cat([q.reshape(L, -1), k.reshape(L, -1), v.reshape(L, -1)], dim=1).contiguous().to(DEV)
        pos = torch.arange(L, dtype=torch.int32, device=DEV)
        ops.rope_cache_write(qkv, torch.empty(L, nH * d, dtype=torch.bfloat16, device=DEV), kp, vp, None, None, pos,
                             torch.full((L,), b, dtype=torch.int32, device=DEV), bt, num_heads=nH, num_kv_heads=nKV,
                             head_dim=d, rotary_dim=0, max_position=L - 1, kv_layout=ops.KV_FRAGMENT)
        if dense:
            refs.append(P.attention_dense(q.double().to(DEV), k.double().to(DEV), v.double().to(DEV), scale, cap, window)[L - n:].cpu())
        else:
            refs.append(P.attention_core(q.double(), k.double(), v.double(), scale, cap, window)[L - n:])
        qs.append(q[L - n:])
    q = torch.cat(qs).reshape(-1, nH * d).to(DEV)
    cu = [0]
    for n in new:
        cu.append(cu[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return q, kp, vp, bt, i32(cu), i32(list(lens)), torch.cat(refs).reshape(-1, nH * d), scale


FRAG_SHAPES = [(6, 2, 64), (4, 4, 64), (8, 4, 256), (4, 1, 128), (3, 3, 128), (32, 16, 128), (16, 1, 256)]


def test_fragment_cache_layout_is_what_the_comment_says():
    nKV, d, L = 2, 64, 70
    kp, vp, bt = paged(L, nKV, d, torch.bfloat16, 1, seed=30)
    k = rnd(L, nKV, d, seed=31, dtype=torch.bfloat16)
    v = rnd(L, nKV, d, seed=32, dtype=torch.bfloat16)
    qkv = torch.cat([torch.zeros(L, d, dtype=torch.bfloat16, device=DEV), k.reshape(L, -1), v.reshape(L, -1)], 1).contiguous()
    ops.rope_cache_write(qkv, torch.empty(L, d, dtype=torch.bfloat16, device=DEV), kp, vp, None, None,
                         torch.arange(L, dtype=torch.int32, device=DEV), torch.zeros(L, dtype=torch.int32, device=DEV), bt,
                         num_heads=1, num_kv_heads=nKV, head_dim=d, rotary_dim=0, max_position=L - 1, kv_layout=ops.KV_FRAGMENT)
    for t, h, e in ((0, 0, 0), (17, 1, 37), (63, 0, 63), (64, 1, 5), (69, 0, 48), (33, 1, 16)):
        page, tp = int(bt[0, t // 64]), t % 64
        kflat, vflat = kp[page, h].reshape(-1), vp[page, h].reshape(-1)
        koff = (((tp // 16) * (d // 32) + e // 32) * 64 + ((e % 32) // 8) * 16 + tp % 16) * 8 + e % 8
        w = tp % 16
        voff = (((tp // 32) * (d // 16) + e // 16) * 64 + (w // 4) * 16 + e % 16) * 8 + (((tp % 32) // 16) * 4 + w % 4)
        assert kflat[koff] == k[t, h, e] and vflat[voff] == v[t, h, e]


@pytest.mark.parametrize("nH,nKV,d", [(3, 2, 64), (8, 4, 256), (2, 1, 128), (1, 1, 32)])
def test_rope_into_the_fragment_cache_layout(nH, nKV, d):
    # rotation and the fragment layout together, every element checked through the layout's formula
    _rope_fragment_case(nH, nKV, d, [70, 3], [0, 62])
    _rope_fragment_case(nH, nKV, d, [290, 3], [0, 62])       # many tokens: the vector kernel


def _rope_fragment_case(nH, nKV, d, lens, starts):
    T = sum(lens)
    qkv = rnd(T, (nH + 2 * nKV) * d, seed=40, dtype=torch.bfloat16)
    pos = torch.tensor([s + i for s, n in zip(starts, lens) for i in range(n)], dtype=torch.int32, device=DEV)
    seq = torch.tensor([b for b, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    kp, vp, bt = paged(320, nKV, d, torch.bfloat16, 2, seed=41)
    theta = 1e4
    ang = torch.arange(300, dtype=D)[:, None] * theta ** (-2.0 * torch.arange(d // 2, dtype=D) / d)
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    q_out = torch.empty(T, nH * d, dtype=torch.bfloat16, device=DEV)
    ops.rope_cache_write(qkv, q_out, kp, vp, cos, sin, pos, seq, bt, num_heads=nH, num_kv_heads=nKV, head_dim=d,
                         rotary_dim=d, max_position=int(pos.max()), kv_layout=ops.KV_FRAGMENT)
    x = qkv.double().cpu()
    q = P.rope_half_split(x[:, :nH * d].view(T, nH, d), pos.cpu(), theta)
    k = P.rope_half_split(x[:, nH * d:(nH + nKV) * d].view(T, nKV, d), pos.cpu(), theta)
    v = x[:, (nH + nKV) * d:].view(T, nKV, d)
    close(q_out.view(T, nH, d), q, 2 ** -5, 2 ** -7)
    e = torch.arange(d)
    for t in range(T):
        page, tp = int(bt[int(seq[t]), int(pos[t]) // 64]), int(pos[t]) % 64
        koff = (((tp // 16) * (d // 32) + e // 32) * 64 + ((e % 32) // 8) * 16 + tp % 16) * 8 + e % 8
        w = tp % 16
        voff = (((tp // 32) * (d // 16) + e // 16) * 64 + (w // 4) * 16 + e % 16) * 8 + (((tp % 32) // 16) * 4 + w % 4)
        for h in range(nKV):
            close(kp[page, h].reshape(-1).cpu()[koff], k[t, h], 2 ** -5, 2 ** -7)
            assert torch.equal(vp[page, h].reshape(-1).cpu()[voff].double(), v[t, h])


def pair_order(nH, nKV, d):
    """Row order of a fused q|k|v projection whose q and k heads have the rotated pairs next to each other."""
    one = torch.stack([torch.arange(d // 2), torch.arange(d // 2) + d // 2], dim=1).flatten()
    heads = torch.arange(nH + nKV)[:, None] * d + one[None, :]
    return torch.cat([heads.flatten(), torch.arange((nH + nKV) * d, (nH + 2 * nKV) * d)])


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("nH,nKV,d,T", [(4, 1, 16, 9), (3, 2, 64, 40), (8, 4, 256, 300), (2, 2, 32, 270)])
@pytest.mark.parametrize("layout", [0, 1])
def test_rope_takes_pairs_next_to_each_other(dt, nH, nKV, d, T, layout):
    # the same rows with the pairs (j, j + d/2) at 2j, 2j + 1 give the same bits (both kernels: few and many tokens)
    if layout == 1 and (dt == "float32" or d % 32):
        pytest.skip("the fragment cache layout is bfloat16 with head sizes in steps of 32")
    qkv = rnd(T, (nH + 2 * nKV) * d, seed=50, dtype=DT[dt])
    pos = torch.arange(T, dtype=torch.int32, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    ang = torch.arange(T, dtype=D)[:, None] * 1e4 ** (-2.0 * torch.arange(d // 2, dtype=D) / d)
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    outs = []
    for inter in (False, True):
        kp, vp, bt = paged(T, nKV, d, DT[dt], 1, seed=51)
        q_out = torch.full((T, nH * d), float("nan"), dtype=DT[dt], device=DEV)
        src = qkv[:, pair_order(nH, nKV, d).to(DEV)].contiguous() if inter else qkv
        ops.rope_cache_write(src, q_out, kp, vp, cos, sin, pos, seq, bt, num_heads=nH, num_kv_heads=nKV, head_dim=d,
                             rotary_dim=d, max_position=T - 1, kv_layout=layout, interleaved=inter)
        outs.append((q_out, kp, vp))
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize("nH,nKV,d,K", [(8, 4, 256, 2304), (3, 1, 64, 96), (4, 2, 128, 320), (2, 2, 16, 72), (16, 16, 128, 64)])
@pytest.mark.parametrize("M", [1, 7, 16, 33, 64, 130, 300, -300, -3100])
@pytest.mark.parametrize("layout", [0, 1])
def test_projection_with_rotation_and_cache_write_as_its_epilogue(nH, nKV, d, K, M, layout):
    if layout == 1 and d % 32:
        pytest.skip("the fragment cache layout takes head sizes in steps of 32")
    runs, M = M < 0, abs(M)
    if M > 1000 and K < 2304:
        pytest.skip("the longest case once")
    N = (nH + 2 * nKV) * d
    x, w = rnd(M, K, seed=60, dtype=torch.bfloat16), rnd(N, K, seed=61, scale=0.1, dtype=torch.bfloat16)
    wf = ops.to_frag16(w[pair_order(nH, nKV, d).to(DEV)].contiguous())
    if runs:
        # two prompts one after the other: the first starts at place 0, so that its tokens come in whole tiles of
        # the cache (the kernels' wide stores), the second at place 5 and at a token that is no multiple of 32
        n_seq, first = 2, (M // 2) // 32 * 32 + 6
        pos = torch.tensor([t if t < first else 5 + t - first for t in range(M)], dtype=torch.int32, device=DEV)
        seq = torch.tensor([1 if t < first else 0 for t in range(M)], dtype=torch.int32, device=DEV)
    else:
        # up to five sequences that start at different places; consecutive tokens go to different sequences
        n_seq, starts = min(M, 5), [0, 60, 100, 7, 33]
        order = torch.randperm(n_seq, generator=torch.Generator().manual_seed(1)).tolist()
        pos = torch.tensor([starts[t % n_seq] + t // n_seq for t in range(M)], dtype=torch.int32, device=DEV)
        seq = torch.tensor([order[t % n_seq] for t in range(M)], dtype=torch.int32, device=DEV)
    lens = [int(pos.max()) + 1]
    ang = torch.arange(max(lens), dtype=D)[:, None] * 1e4 ** (-2.0 * torch.arange(d // 2, dtype=D) / d)
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    # The separate kernels first; between 33 and 64 tokens with both of the product's kernels, since the fused call
    # takes the streaming or the tiled one by its rule there (they add up the inner dimension in different orders).
    res = []
    cases = [(False, False, ops.LINEAR_AUTO)] + ([(False, False, ops.LINEAR_MFMA)] if 32 < M <= 64 else [])
    cases += [(True, frag_in, None) for frag_in in ((False, True) if K % 32 == 0 else (False,))]
    for fused, frag_in, variant in cases:
        kp, vp, bt = paged(max(lens), nKV, d, torch.bfloat16, n_seq, seed=62)
        q_out = torch.full((M, nH * d), float("nan"), dtype=torch.bfloat16, device=DEV)
        if fused:
            xin = acts_to_fragments(x) if frag_in else x
            ops.linear_rope_cache(xin, wf, q_out, kp, vp, cos, sin, pos, seq, bt, k_in=K, num_heads=nH, num_kv_heads=nKV,
                                  head_dim=d, max_position=max(lens) - 1, kv_layout=layout, rows=M,
                                  x_layout=ops.LAYOUT_FRAG16 if frag_in else ops.LAYOUT_ROW)
        else:
            qkv = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            ops.linear(x, wf, qkv, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, variant=variant, full_precision=False)
            ops.rope_cache_write(qkv, q_out, kp, vp, cos, sin, pos, seq, bt, num_heads=nH, num_kv_heads=nKV, head_dim=d,
                                 rotary_dim=d, max_position=max(lens) - 1, kv_layout=layout, interleaved=True)
        res.append((fused, (q_out, kp, vp)))
    separate = [r for f, r in res if not f]
    for f, other in res:
        if f:
            assert any(all(torch.equal(a, b) for a, b in zip(ref, other)) for ref in separate)
    res = [r for _, r in res]
    # and the separate kernels against the plain formulas, from the rows in their plain order
    qkv_ref = x.double().cpu() @ w.double().cpu().T
    qkv_ref = qkv_ref.to(torch.bfloat16).double()
    q_ref = P.rope_half_split(qkv_ref[:, :nH * d].view(M, nH, d), pos.cpu(), 1e4)
    close(res[0][0].view(M, nH, d), q_ref, 2 ** -5, 2 ** -6)


@pytest.mark.parametrize("nH,nKV,d", FRAG_SHAPES)
@pytest.mark.parametrize("cap,window", [(None, None), (5.0, 50), (50.0, 7), (2.0, 64)])
def test_attention_mfma_prompts(nH, nKV, d, cap, window):
    for lens, new in (((5, 130, 66), (5, 130, 66)), ((150, 64, 33), (20, 3, 33)), ((300,), (300,))):
        q, kp, vp, bt, cu, ctx, ref, scale = frag_case(nH, nKV, d, lens, new, cap, window, seed=3)
        for variant in (ops.PREFILL_TILES, ops.PREFILL_SPLIT, ops.PREFILL_SHARED4, ops.PREFILL_SHARED8, ops.PREFILL_SHARED4X2, ops.PREFILL_AUTO):
            out = torch.full_like(q, float("nan"))
            ops.attention_prefill(q, kp, vp, out, cu, ctx, bt, num_heads=nH, n_seqs=len(lens), max_new=max(new),
                                  max_context=max(lens), scale=scale, softcap=cap, window=window, variant=variant)
            close(out, ref, 2e-2)
            if (nH * d) % 32 == 0 and variant != ops.PREFILL_AUTO:
                # output in fragment order for the projection that follows: the same bits, elsewhere
                T = q.shape[0]
                flat = torch.full(((-(-T // 16) * 16) * nH * d,), float("nan"), dtype=torch.bfloat16, device=DEV)
                ops.attention_prefill(q, kp, vp, flat, cu, ctx, bt, num_heads=nH, n_seqs=len(lens), max_new=max(new),
                                      max_context=max(lens), scale=scale, softcap=cap, window=window, variant=variant,
                                      out_layout=ops.LAYOUT_FRAG16)
                assert torch.equal(acts_from_fragments(flat, T, nH * d), out.cpu())


@pytest.mark.parametrize("nH,nKV,d", [(8, 4, 256), (32, 16, 128), (6, 2, 64), (8, 8, 128), (3, 3, 128)])   # (3, 3): see below
@pytest.mark.parametrize("cap,window", [(50.0, None), (4.0, 1000)])
def test_attention_mfma_prompts_that_make_more_blocks_than_cus(nH, nKV, d, cap, window):
    """Long prompts: the kernels whose waves share keys through LDS then have more blocks than the chip has CUs and
    deal the kv heads to the XCDs (blocks that read the same keys meet in one L2); with 1, 2, 4, 8 and 16 kv heads
    times passes, and 6, a number that fits neither way (dealt plainly); whole prompts and a prompt on a cached prefix."""
    cases = [((1300, 1100), (1300, 1100)), ((2500,), (1200,))]
    if nKV == 3:
        cases = [((2304, 2304), (2304, 2304))]       # 288 blocks of the one or two kv-head passes of (4, 1) and (4, 2) heads
        nH, nKV = 4, 1 if cap == 4.0 else 2
    for lens, new in cases:
        q, kp, vp, bt, cu, ctx, ref, scale = frag_case(nH, nKV, d, lens, new, cap, window, seed=4, dense=True)
        for variant in (ops.PREFILL_SHARED4, ops.PREFILL_SHARED8, ops.PREFILL_SHARED4X2, ops.PREFILL_AUTO):
            out = torch.full_like(q, float("nan"))
            ops.attention_prefill(q, kp, vp, out, cu, ctx, bt, num_heads=nH, n_seqs=len(lens), max_new=max(new),
                                  max_context=max(lens), scale=scale, softcap=cap, window=window, variant=variant)
            close(out, ref, 2e-2)


@pytest.mark.parametrize("nH,nKV,d", FRAG_SHAPES)
@pytest.mark.parametrize("cap,window", [(None, None), (5.0, 50), (50.0, 7), (2.0, 64)])
def test_attention_mfma_single_tokens(nH, nKV, d, cap, window):
    lens = (200, 1, 77, 64, 65, 33, 700)
    q, kp, vp, bt, cu, ctx, ref, scale = frag_case(nH, nKV, d, lens, (1,) * len(lens), cap, window, seed=4)
    for splits in (None, 1, 2, 5, 16):
        out = torch.full_like(q, float("nan"))
        ops.attention_decode(q, kp, vp, out, ctx, bt, num_heads=nH, max_context=max(lens), scale=scale, softcap=cap,
                             window=window, splits=splits)
        close(out, ref, 2e-2)
    # output in fragment order for the projection that follows: the same bits, elsewhere
    if (nH * d) % 32 == 0:
        ops.attention_decode(q, kp, vp, out, ctx, bt, num_heads=nH, max_context=max(lens), scale=scale, softcap=cap, window=window)
        flat = torch.full((16 * nH * d,), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.attention_decode(q, kp, vp, flat, ctx, bt, num_heads=nH, max_context=max(lens), scale=scale, softcap=cap,
                             window=window, out_layout=ops.LAYOUT_FRAG16)
        assert torch.equal(acts_from_fragments(flat, len(lens), nH * d), out.cpu())
    # the prompt kernels on single tokens give the same
    for variant in (ops.PREFILL_TILES, ops.PREFILL_SPLIT, ops.PREFILL_SHARED4, ops.PREFILL_SHARED8, ops.PREFILL_SHARED4X2):
        out = torch.full_like(q, float("nan"))
        ops.attention_prefill(q, kp, vp, out, cu, ctx, bt, num_heads=nH, n_seqs=len(lens), max_new=1, max_context=max(lens),
                              scale=scale, softcap=cap, window=window, variant=variant)
        close(out, ref, 2e-2)


@pytest.mark.parametrize("nH,nKV,d", FRAG_SHAPES)
@pytest.mark.parametrize("N", [2304, 80])
def test_output_projection_that_combines_the_key_splits_itself(nH, nKV, d, N):
    """Single-token attention may leave its key splits uncombined; the output projection then combines them in its
    prologue.  Against the separate kernels (combine, then project) and against the plain formula, for 1 to 16
    sequences, 2 to 16 splits, slices that cover several heads, one head, or a part of one."""
    lens = (200, 1, 77, 64, 65, 33, 700, 129, 12, 300, 5, 90, 450, 31, 64, 2)
    w = rnd(N, nH * d, seed=70, scale=0.1, dtype=torch.bfloat16)
    wf = ops.to_frag16(w)
    for B, splits in ((16, 5), (7, 2), (1, 16), (8, 8), (3, 9)):
        q, kp, vp, bt, cu, ctx, ref, scale = frag_case(nH, nKV, d, lens[:B], (1,) * B, 5.0, 50, seed=4)
        slices = ops.linear_parts_slices(B, N, nH, d, splits)
        assert slices > 0
        out = torch.full_like(q, float("nan"))
        ops.attention_decode(q, kp, vp, out, ctx, bt, num_heads=nH, max_context=max(lens[:B]), scale=scale, softcap=5.0,
                             window=50, splits=splits)
        parts, _ = ops.attention_decode(q, kp, vp, None, ctx, bt, num_heads=nH, max_context=max(lens[:B]), scale=scale,
                                        softcap=5.0, window=50, splits=splits)
        y = torch.full((slices, B, N), float("nan"), dtype=torch.float32, device=DEV)
        ops.linear_parts(parts, splits, wf, y, num_heads=nH, head_dim=d)
        separate = torch.empty(B, N, dtype=torch.float32, device=DEV)
        ops.linear(out, wf, separate, n_out=N, k_in=nH * d, layout=ops.LAYOUT_FRAG16, full_precision=False)
        close(y.sum(0), separate, 2e-3, 1e-3)                # the same rounded activations, other orders of the sums
        close(y.sum(0), ref.double().reshape(B, -1).cpu() @ w.double().cpu().T, 4e-2 * math.sqrt(nH * d / 64), 2 ** -6)
    assert ops.linear_parts_slices(17, N, nH, d, 4) == 0 and ops.linear_parts_slices(4, N, nH, d, 1) == 0
    assert ops.linear_parts_slices(4, N, nH, d, 17) == 0
    with pytest.raises(ops.HipLibraryError):
        ops.attention_decode(q, kp, vp, None, ctx, bt, num_heads=nH, max_context=max(lens), scale=scale, softcap=5.0,
                             window=50, splits=1)


def test_many_heads_and_a_narrow_output_keep_the_slices_few():
    """40 heads of 64 and 24 output features: the rule for the blocks would cut the inner dimension into 80 slices
    of one k-tile, more partial results than the add + norm that follows sums; it stops at 16."""
    nH, nKV, d, N, B, splits = 40, 5, 64, 24, 3, 4
    for n_out in (N, 130, 2304):
        for M in (1, B, 16):
            assert 0 <= ops.linear_parts_slices(M, n_out, nH, d, splits) <= 16
    assert ops.linear_parts_slices(B, N, 128, 256, splits) == 0          # an inner dimension of 32,768: not covered
    lens = (150, 70, 9)
    w = rnd(N, nH * d, seed=71, scale=0.1, dtype=torch.bfloat16)
    wf = ops.to_frag16(w)
    q, kp, vp, bt, cu, ctx, ref, scale = frag_case(nH, nKV, d, lens, (1,) * B, None, None, seed=6)
    slices = ops.linear_parts_slices(B, N, nH, d, splits)
    assert slices > 0
    parts, _ = ops.attention_decode(q, kp, vp, None, ctx, bt, num_heads=nH, max_context=max(lens), scale=scale, softcap=None,
                                    window=None, splits=splits)
    y = torch.full((slices, B, N), float("nan"), dtype=torch.float32, device=DEV)
    ops.linear_parts(parts, splits, wf, y, num_heads=nH, head_dim=d)
    close(y.sum(0), ref.double().reshape(B, -1).cpu() @ w.double().cpu().T, 4e-2 * math.sqrt(nH * d / 64), 2 ** -6)
    # the partial results go through the fused add + norm as the block does it
    resid = rnd(B, N, seed=72, dtype=torch.float32)
    w_post = rnd(N, seed=73, dtype=torch.float32)
    want = resid.double() + P.rms_norm(y.double().sum(0), w_post.double(), 1e-6)
    ops.add_norm(resid, y, w_post, None, None, eps_post=1e-6, off_post=1.0, n_partials=slices, full_precision=False)
    close(resid, want, 1e-4, 1e-5)


def test_attention_mfma_far_key_and_window_edge():
    nH, nKV, d, L = 4, 2, 64, 700
    def far(b, q, k, v):
        k[3] = 0; k[3, :, 0] = 40.0
        q[L - 1] = 0; q[L - 1, :, 0] = 40.0
    q, kp, vp, bt, cu, ctx, ref, scale = frag_case(nH, nKV, d, (L,), (1,), None, None, seed=5, crafted=far)
    for fn in ("decode", ops.PREFILL_TILES, ops.PREFILL_SPLIT, ops.PREFILL_SHARED4, ops.PREFILL_SHARED8, ops.PREFILL_SHARED4X2):
        out = torch.full_like(q, float("nan"))
        if fn == "decode":
            ops.attention_decode(q, kp, vp, out, ctx, bt, num_heads=nH, max_context=L, scale=scale, softcap=None, window=None)
        else:
            ops.attention_prefill(q, kp, vp, out, cu, ctx, bt, num_heads=nH, n_seqs=1, max_new=1, max_context=L, scale=scale,
                                  softcap=None, window=None, variant=fn)
        close(out, ref, 2e-2)
        assert (out.view(nH, d)[0].double().cpu() - ref.view(nH, d)[0]).abs().max() < 2e-2 and ref.view(nH, d)[0].abs().max() > 0.1
    for where, seen in ((L - 101, False), (L - 100, True)):
        def edge(b, q, k, v, where=where):
            k[where] = 0; k[where, :, 0] = 40.0; v[where] = 7.0
            q[L - 1] = 0; q[L - 1, :, 0] = 40.0
        q, kp, vp, bt, cu, ctx, ref, scale = frag_case(nH, nKV, d, (L,), (1,), None, 100, seed=6, crafted=edge)
        for fn in ("decode", ops.PREFILL_TILES, ops.PREFILL_SPLIT, ops.PREFILL_SHARED4, ops.PREFILL_SHARED8, ops.PREFILL_SHARED4X2):
            out = torch.full_like(q, float("nan"))
            if fn == "decode":
                ops.attention_decode(q, kp, vp, out, ctx, bt, num_heads=nH, max_context=L, scale=scale, softcap=None, window=100)
            else:
                ops.attention_prefill(q, kp, vp, out, cu, ctx, bt, num_heads=nH, n_seqs=1, max_new=1, max_context=L,
                                      scale=scale, softcap=None, window=100, variant=fn)
            close(out, ref, 2e-2)
            assert (abs(float(out[0, 0]) - 7.0) < 5e-2) == seen


def test_attention_mfma_refuses_other_head_sizes():
    assert ops.attention_mfma_supported(256) and not ops.attention_mfma_supported(24) and not ops.attention_mfma_supported(96)
    kp = torch.zeros(2, 1, 64, 96, dtype=torch.bfloat16, device=DEV)
    q = torch.zeros(1, 96, dtype=torch.bfloat16, device=DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    with pytest.raises(ops.HipLibraryError, match="head_dim 96 is not covered"):
        ops.attention_decode(q, kp, kp, q.clone(), i32([5]), i32([[1]]), num_heads=1, max_context=5, scale=1.0, softcap=None, window=None)


def test_linear_mfma_vocabulary_sized_output():
    # the output head's shape: a quarter of a million rows, a width that is no power of two
    N, K = 256000, 96
    w = rnd(N, K, seed=40, scale=0.1, dtype=torch.bfloat16)
    wf = ops.to_frag16(w)
    for M in (1, 8, 64, 100):
        x = rnd(M, K, seed=41, dtype=torch.bfloat16)
        y = torch.empty(M, N, dtype=torch.float32, device=DEV)
        ops.linear(x, wf, y, n_out=N, k_in=K, layout=ops.LAYOUT_FRAG16, epilogue=ops.EPI_SOFTCAP, epi_param=30.0, full_precision=False)
        close(y, 30.0 * torch.tanh((x.double() @ w.double().T) / 30.0), 2e-3)
