"""Decode and prefill throughput of the Gemma 2 shapes with random weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of a batch of 8 sequences that were prefilled with 2,048-token prompts;
by default the timed steps run the context from 2,048 out to 4,096.  The printed line also holds the
prefill of one 2,048-token prompt (and of prompts of 8,192, 512 and 128 tokens), the decode step's memory roofline (at the
mean context of the timed steps), and decode throughput at batch 1 and 64 over the same range, each with
its roofline.  Beside the published peaks the line gives what this GPU itself reaches (`peak_measured`: a
device-to-device copy and a large bfloat16 matrix product of the vendor library) and, under `shapes`, shorter runs
of the other configurations: the 2B shape at contexts from 8,000, 16 unequal prompts at the 9B shape, and 8 prompts
of 6,000 tokens, past the window, at the 27B shape.

Other runs of the same program:
    python bench.py --preset 9b --batch 16 --prompt-lens uniform:64:2048 --steps 256 --points "" --shapes ""
        16 prompts of unequal, seeded lengths in ragged steps, then 256 decode steps
    python bench.py --preset 27b --batch 8 --prompt 6000 --context 8192 --steps 128 --points "" --shapes ""
        8 prompts of 6,000 tokens, past the window of 4,096, then 128 decode steps
"""
import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

PEAK_HBM_GBS = 8000.0                       # MI355X HBM3E
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def decode_bytes(cfg, weight_bytes, contexts, elem):
    """Bytes a decode step has to read: every weight once, and the keys and values of the live requests
    (a sliding layer reads at most its window of them)."""
    kv = 0
    for ctx in contexts:
        for i in range(cfg.num_hidden_layers):
            w = cfg.layer_window(i)
            keys = ctx if w is None else min(ctx, w)
            kv += 2 * keys * cfg.kv_dim * elem
    return weight_bytes + kv


def prefill_flops(cfg, T, n_logit_rows=1):
    H, Q, KV, I = cfg.hidden_size, cfg.q_dim, cfg.kv_dim, cfg.intermediate_size
    per_layer = 2 * T * (H * (Q + 2 * KV) + Q * H + 3 * H * I)
    attn = 0
    for i in range(cfg.num_hidden_layers):
        w = cfg.layer_window(i)
        pairs = T * (T + 1) // 2 if not w or w >= T else w * (w + 1) // 2 + (T - w) * w
        attn += 4 * cfg.num_attention_heads * cfg.head_dim * pairs
    return cfg.num_hidden_layers * per_layer + attn + 2 * n_logit_rows * H * cfg.vocab_size


def prompt_lengths(spec, batch, prompt, seed=0):
    """--prompt-lens: 'uniform:LO:HI' draws each sequence's prompt length from [LO, HI] (seeded); a list
    'a,b,c' gives them; nothing gives --prompt to every sequence."""
    import random
    if not spec:
        return [prompt] * batch
    if spec.startswith("uniform:"):
        lo, hi = (int(x) for x in spec.split(":")[1:3])
        rng = random.Random(seed)
        return [rng.randint(lo, hi) for _ in range(batch)]
    lens = [int(x) for x in spec.split(",")]
    if len(lens) != batch:
        raise SystemExit(f"--prompt-lens lists {len(lens)} lengths for a batch of {batch}")
    return lens


def measured_peaks():
    """What this GPU reaches by itself, beside the published peaks: a device-to-device copy of 2 GB (bytes read
    plus bytes written over its time) and an 8,192-cubed bfloat16 matrix product of the vendor library, each the
    median of five by HIP events.  Neither is on the product path."""
    import torch
    out = {}

    def median_ms(fn, n=5):
        fn()
        ts = []
        for _ in range(n):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b))
        return sorted(ts)[n // 2]

    src = torch.empty(1 << 30, dtype=torch.int16, device="cuda")
    dst = torch.empty_like(src)
    ms = median_ms(lambda: dst.copy_(src))
    out["copy_gbs"] = round(2 * src.numel() * 2 / (ms / 1e3) / 1e9, 1)
    del src, dst
    a = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
    ms = median_ms(lambda: torch.matmul(a, b))
    out["bf16_matmul_tflops"] = round(2 * 8192 ** 3 / (ms / 1e3) / 1e12, 1)
    del a, b
    torch.cuda.empty_cache()
    return out


class Run:
    """One model shape with random weights and the measurements on it."""

    def __init__(self, preset, layers, dtype, ids_through_host=False):
        import torch
        import alice_llm_amd as alice
        self.torch, self.alice = torch, alice
        raw = alice.preset(preset)
        self.full_layers = raw["num_hidden_layers"]
        if layers:
            raw["num_hidden_layers"] = layers
        self.cfg = alice.config_from_dict(raw)
        self.dtype = dtype
        self.elem = 2 if dtype == "bfloat16" else 4
        self.short = "bf16" if dtype == "bfloat16" else "fp32"
        self.ids_through_host = ids_through_host
        t0 = time.time()
        self.model = alice.Model.random(self.cfg, seed=0, dtype=dtype, fast=True)
        self.weight_bytes = self.model.lm.weight_bytes()
        print(f"[bench] {preset}: model built in {time.time() - t0:.1f} s, weights {self.weight_bytes / 1e9:.2f} GB",
              file=sys.stderr, flush=True)
        self.gen = torch.Generator().manual_seed(0)
        self.gpu_ms = None

    def prompts(self, lens):
        return [self.torch.randint(0, self.cfg.vocab_size, (n,), generator=self.gen).tolist() for n in lens]

    def decode(self, lens, steps, warmup, context=0):
        """Prefill prompts of these lengths (in the generation loop's ragged steps), then time `steps` decode steps
        (greedy, tokens fed back).  Returns the time and every sequence's context at the first and after the
        last timed step."""
        torch, alice, cfg = self.torch, self.alice, self.cfg
        from alice_llm_amd.hip import ops
        batch = len(lens)
        room = [max(n + warmup + steps, context) for n in lens]
        if max(n + warmup + steps for n in lens) > cfg.max_position_embeddings:
            raise SystemExit(f"prompt + warmup + steps reach beyond the model's {cfg.max_position_embeddings} positions")
        eng = self.model.engine(seq_lens=room, max_seqs=batch)
        slots = eng.open(batch)
        ps = self.prompts(lens)
        # the prompts run as the generation loop runs them: ragged steps of at most its token budget each
        ids = ops.argmax(alice.run_prompt_steps(eng, slots, ps)).tolist()
        # Decode steps as the library's own generation loop runs them: the chosen ids go from the sampling kernel
        # to the next step on the device, and the host queues step n + 1 before it reads step n's ids (through a
        # pinned buffer and an event), so it is one step ahead and no further.
        pending = []

        def one(ids):
            if self.ids_through_host:
                return ops.argmax(eng.step(slots, [[t_] for t_ in ids], "last")).tolist()
            out = ops.argmax(eng.step(slots, ids, "last"))
            host = torch.empty(out.shape, dtype=out.dtype, pin_memory=True)
            host.copy_(out, non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
            pending.append((ev, host))
            if len(pending) > 1:
                ev0, host0 = pending.pop(0)
                ev0.synchronize()
                host0.tolist()                                   # where a loop would look for stop tokens
            return out

        if not self.ids_through_host:
            ids = torch.tensor(ids, dtype=torch.int32, device="cuda")
        for _ in range(warmup):
            ids = one(ids)
        ctx0 = [eng.length(s) for s in slots]
        torch.cuda.synchronize()
        pending.clear()
        t = time.perf_counter()
        for _ in range(steps):
            ids = one(ids)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        ctx1 = [eng.length(s) for s in slots]
        # The GPU's own time for a step: the last captured step replayed back to back with nothing of the host
        # between the replays (it writes the same cache places again and again).  What the timed steps took
        # beyond that is the host's: bookkeeping, the copy of the step's integers, reading the chosen tokens.
        self.gpu_ms = None
        captured = [g for g in eng._graphs.values() if g.graph is not None]
        if captured:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(20):
                captured[-1].graph.replay()
            b.record()
            torch.cuda.synchronize()
            self.gpu_ms = a.elapsed_time(b) / 20
        eng.close(slots)
        del eng
        torch.cuda.empty_cache()
        return dt, ctx0, ctx1

    def roofline(self, dt, steps, ctx0, ctx1):
        mids = [(a + b) // 2 for a, b in zip(ctx0, ctx1)]
        achieved = decode_bytes(self.cfg, self.weight_bytes, mids, self.elem) / (dt / steps) / 1e9
        return {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(achieved / PEAK_HBM_GBS, 4)}

    def prefill(self, T, repeats=5):
        """One prompt of T tokens through one step: the median of `repeats` timings by HIP events (after one
        untimed pass), the wall clock's minimum beside it."""
        torch = self.torch
        eng = self.model.engine(seq_lens=[T], max_seqs=1)
        p = self.prompts([T])
        gpu, wall = [], []
        for it in range(repeats + 1):
            s = eng.open(1)
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t = time.perf_counter()
            a.record()
            eng.step(s, p, "last")
            b.record()
            torch.cuda.synchronize()
            if it:
                wall.append((time.perf_counter() - t) * 1e3)
                gpu.append(a.elapsed_time(b))
            eng.close(s)
        ms = sorted(gpu)[len(gpu) // 2]
        fl = prefill_flops(self.cfg, T)
        # frac: the step's flops over the matrix cores' peak; hbm_frac: the weights, which every step reads once,
        # over the memory's peak (what bounds a prompt of a few hundred tokens)
        out = {"value": round(T / (ms / 1e3), 1), "tokens": T, "ms": round(ms, 3),
               "frac": round(fl / (ms / 1e3) / PEAK_FLOPS[self.short], 4),
               "hbm_frac": round(self.weight_bytes / (ms / 1e3) / 1e9 / PEAK_HBM_GBS, 4),
               "timing": f"median of {repeats} by HIP events", "wall_ms_min": round(min(wall), 3)}
        del eng
        torch.cuda.empty_cache()
        return out

    def close(self):
        del self.model
        self.torch.cuda.empty_cache()


SHAPES = {
    "2b-ctx8k": dict(preset="2b", batches=(8, 64), prompt=8000, lens="", steps=20),
    "9b-unequal": dict(preset="9b", batches=(16,), prompt=0, lens="uniform:64:2048", steps=64),
    "27b-6000": dict(preset="27b", batches=(8,), prompt=6000, lens="", steps=32),
}


def shape_run(name, dtype):
    """A shorter run of another configuration, every figure with its configuration beside it."""
    spec = SHAPES[name]
    run = Run(spec["preset"], None, dtype)
    cfg = run.cfg
    out = {"model": f"gemma2-{spec['preset']}", "layers": cfg.num_hidden_layers, "weights_gb": round(run.weight_bytes / 1e9, 2),
           "steps": spec["steps"], "warmup": 3}
    for b in spec["batches"]:
        lens = prompt_lengths(spec["lens"], b, spec["prompt"])
        dt, c0, c1 = run.decode(lens, spec["steps"], 3)
        roof = run.roofline(dt, spec["steps"], c0, c1)
        out[f"decode_b{b}"] = {"tok_s": round(b * spec["steps"] / dt, 1), "ms_per_step": round(dt / spec["steps"] * 1e3, 4),
                               "prompt_len_min": min(lens), "prompt_len_max": max(lens),
                               "context_start": int(round(sum(c0) / len(c0))), "context_end": int(round(sum(c1) / len(c1))),
                               "roofline_gbs": roof["achieved"], "roofline_frac": roof["frac"]}
        print(f"[bench] {name} decode_b{b}: {out[f'decode_b{b}']}", file=sys.stderr, flush=True)
    if spec["preset"] != "2b":
        pf = run.prefill(2048, repeats=3)
        out["prefill_2048"] = {"tok_s": pf["value"], "ms": pf["ms"], "frac": pf["frac"]}
    run.close()
    return out


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2048)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--preset", default="2b")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the preset (both numbers are reported)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--prompt-lens", default="", help="unequal prompts: 'uniform:LO:HI' (seeded) or a list 'a,b,c'")
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64", help="other batch sizes to measure decode at ('' for none)")
    ap.add_argument("--point-steps", type=int, default=None, help="steps for the other batch sizes (default: --steps)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--ids-through-host", action="store_true",
                    help="read every step's chosen ids on the host before the next step is queued (the loop with an observer)")
    ap.add_argument("--prefill-tokens", default="2048,8192,512,128", help="prompt lengths whose prefill is timed (the first is the headline's)")
    ap.add_argument("--shapes", default=",".join(SHAPES),
                    help="shorter runs of other configurations, reported under 'shapes' ('' for none)")
    ap.add_argument("--no-peaks", action="store_true", help="skip the measurement of this GPU's own copy and matrix-product rates")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2

    import torch
    torch.cuda.set_device(0)
    run = Run(args.preset, args.layers, args.dtype, args.ids_through_host)
    cfg, short = run.cfg, run.short

    # ---- prefill of one prompt (2,048 tokens for the headline; other lengths beside it)
    prefills = {}
    if not args.no_prefill:
        for T in [int(x) for x in args.prefill_tokens.split(",") if x]:
            if T > cfg.max_position_embeddings:
                continue
            prefills[T] = run.prefill(T)
            print(f"[bench] prefill {prefills[T]}", file=sys.stderr, flush=True)
    prefill_keys = list(prefills)

    # ---- the headline: decode at the default batch
    lens = prompt_lengths(args.prompt_lens, args.batch, args.prompt)
    context = 0 if args.prompt_lens else args.context
    dt, ctx0, ctx1 = run.decode(lens, args.steps, args.warmup, context)
    ms_step = dt / args.steps * 1e3
    gpu_ms_step = run.gpu_ms
    value = args.batch * args.steps / dt
    points, point_rooflines = {}, {}
    for b in [int(x) for x in args.points.split(",") if x]:
        psteps = args.point_steps or args.steps
        pdt, p0, p1 = run.decode(prompt_lengths(args.prompt_lens, b, args.prompt), psteps, args.warmup, context)
        points[f"decode_b{b}"] = round(b * psteps / pdt, 1)
        point_rooflines[f"decode_b{b}"] = dict(run.roofline(pdt, psteps, p0, p1), ms_per_step=round(pdt / psteps * 1e3, 4))
        print(f"[bench] decode_b{b}: {points[f'decode_b{b}']} tok/s, {point_rooflines[f'decode_b{b}']}", file=sys.stderr, flush=True)
    roof = run.roofline(dt, args.steps, ctx0, ctx1)
    weight_bytes, full_layers = run.weight_bytes, run.full_layers
    prefill_fl = {T: prefill_flops(cfg, T) for T in prefills}
    run.close()

    shapes = {}
    for name in [s for s in args.shapes.split(",") if s]:
        if name not in SHAPES:
            raise SystemExit(f"--shapes: unknown '{name}'; known: {sorted(SHAPES)}")
        t0 = time.time()
        shapes[name] = shape_run(name, args.dtype)
        print(f"[bench] shape {name} took {time.time() - t0:.1f} s", file=sys.stderr, flush=True)

    # this GPU's own rates last, so that their heat is not in the figures above; the fractions of them are added here
    peaks = {} if args.no_peaks else measured_peaks()
    if peaks:
        print(f"[bench] measured on this GPU: {peaks}", file=sys.stderr, flush=True)
        for r in [roof] + list(point_rooflines.values()):
            r["frac_of_measured_copy"] = round(r["achieved"] / peaks["copy_gbs"], 4)
        if short == "bf16":
            for T, pf in prefills.items():
                pf["frac_of_measured_matmul"] = round(prefill_fl[T] / (pf["ms"] / 1e3) / 1e12 / peaks["bf16_matmul_tflops"], 4)

    mean = lambda xs: int(round(sum(xs) / len(xs)))
    line = {
        "metric": (f"decode tok/s @ batch {args.batch}, Gemma-2-{args.preset.upper()} {short} "
                   f"(points: batch {'/'.join(str(int(x)) for x in args.points.split(',') if x) or '-'}; "
                   f"prefill tok/s @ {prefill_keys[0] if prefill_keys else 0:,} tok)"),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "gpu_ms_per_step": round(gpu_ms_step, 4) if gpu_ms_step else None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic (uniform random token ids, random weights N(0, 0.02))",
        "config": {"model": f"gemma2-{args.preset}", "global_batch": args.batch, "seq_len": max(args.context, max(ctx1)),
                   "prompt_len": mean(lens), "prompt_lens": args.prompt_lens or "equal",
                   "prompt_len_min": min(lens), "prompt_len_max": max(lens),
                   "context_start": mean(ctx0), "context_end": mean(ctx1), "parallelism": "single-gpu",
                   "layers": cfg.num_hidden_layers, "layers_of_model": full_layers, "hidden": cfg.hidden_size,
                   "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "sliding_window": cfg.sliding_window,
                   "weights_gb": round(weight_bytes / 1e9, 3)},
        "prefill": prefills[prefill_keys[0]] if prefill_keys else None,
        "roofline": roof,
        "points": points,
        "point_rooflines": point_rooflines,
    }
    for T in prefill_keys[1:]:
        line[f"prefill_{T}"] = prefills[T]
    if peaks:
        line["peak_measured"] = peaks
    if shapes:
        line["shapes"] = shapes
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
