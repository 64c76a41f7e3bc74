"""Decode and prefill throughput of the Gemma 2 shapes with random weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of a batch of 8 sequences that were prefilled with 2,048-token prompts;
by default the timed steps run the context from 2,048 out to 4,096.  The printed line also holds the
prefill of one 2,048-token prompt (and of prompts of 8,192, 512 and 128 tokens), the decode step's memory roofline (at the
mean context of the timed steps), and decode throughput at batch 1 and 64 over the same range, each with
its roofline.

Other runs of the same program:
    python bench.py --preset 9b --batch 16 --prompt-lens uniform:64:2048 --steps 256 --points ""
        16 prompts of unequal, seeded lengths in one ragged step, then 256 decode steps
    python bench.py --preset 27b --batch 8 --prompt 6000 --context 8192 --steps 128 --points ""
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
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2

    import torch
    import alice_llm_amd as alice
    from alice_llm_amd.hip import ops

    torch.cuda.set_device(0)
    raw = alice.preset(args.preset)
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    cfg = alice.config_from_dict(raw)
    t0 = time.time()
    model = alice.Model.random(cfg, seed=0, dtype=args.dtype, fast=True)
    weight_bytes = model.lm.weight_bytes()
    print(f"[bench] model built in {time.time() - t0:.1f} s, weights {weight_bytes / 1e9:.2f} GB", file=sys.stderr, flush=True)
    elem = 2 if args.dtype == "bfloat16" else 4
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    gen = torch.Generator().manual_seed(0)

    def prompts(lens):
        return [torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist() for n in lens]

    def sync():
        torch.cuda.synchronize()

    def decode_run(lens, steps, warmup):
        """Prefill prompts of these lengths (in the generation loop's ragged steps), then time `steps` decode steps
        (greedy, tokens fed back).  Returns the time and every sequence's context at the first and after the
        last timed step."""
        batch = len(lens)
        room = [max(n + warmup + steps, args.context if not args.prompt_lens else 0) for n in lens]
        if max(n + warmup + steps for n in lens) > cfg.max_position_embeddings:
            raise SystemExit(f"prompt + warmup + steps reach beyond the model's {cfg.max_position_embeddings} positions")
        eng = model.engine(seq_lens=room, max_seqs=batch)
        slots = eng.open(batch)
        ps = prompts(lens)
        # the prompts run as the generation loop runs them: ragged steps of at most its token budget each
        ids = ops.argmax(alice.run_prompt_steps(eng, slots, ps)).tolist()
        print(f"[bench] prefilled {batch} prompts in {len(alice.plan_prompt_steps(lens, alice.engine.generate.MAX_STEP_TOKENS))} steps",
              file=sys.stderr, flush=True)
        # Decode steps as the library's own generation loop runs them: the chosen ids go from the sampling kernel
        # to the next step on the device, and the host queues step n + 1 before it reads step n's ids (through a
        # pinned buffer and an event), so it is one step ahead and no further.
        pending = []

        def one(ids):
            if args.ids_through_host:
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

        if not args.ids_through_host:
            ids = torch.tensor(ids, dtype=torch.int32, device="cuda")
        for _ in range(warmup):
            ids = one(ids)
        ctx0 = [eng.length(s) for s in slots]
        sync()
        pending.clear()
        t = time.perf_counter()
        for _ in range(steps):
            ids = one(ids)
        sync()
        dt = time.perf_counter() - t
        ctx1 = [eng.length(s) for s in slots]
        # The GPU's own time for a step: the last captured step replayed back to back with nothing of the host
        # between the replays (it writes the same cache places again and again).  What the timed steps took
        # beyond that is the host's: bookkeeping, the copy of the step's integers, reading the chosen tokens.
        decode_run.gpu_ms = None
        captured = [g for g in eng._graphs.values() if g.graph is not None]
        if captured:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(20):
                captured[-1].graph.replay()
            b.record()
            sync()
            decode_run.gpu_ms = a.elapsed_time(b) / 20
        eng.close(slots)
        del eng
        torch.cuda.empty_cache()
        return dt, ctx0, ctx1

    def roofline(dt, steps, ctx0, ctx1):
        mids = [(a + b) // 2 for a, b in zip(ctx0, ctx1)]
        achieved = decode_bytes(cfg, weight_bytes, mids, elem) / (dt / steps) / 1e9
        return {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(achieved / PEAK_HBM_GBS, 4)}

    # ---- prefill of one prompt (2,048 tokens for the headline; a second length beside it)
    prefills = {}
    if not args.no_prefill:
        for T in [int(x) for x in args.prefill_tokens.split(",") if x]:
            if T > cfg.max_position_embeddings:
                continue
            eng = model.engine(seq_lens=[T], max_seqs=1)
            p = prompts([T])
            times = []
            for it in range(6):
                s = eng.open(1)
                sync()
                t = time.perf_counter()
                eng.step(s, p, "last")
                sync()
                times.append(time.perf_counter() - t)
                eng.close(s)
            ms = min(times[1:]) * 1e3
            fl = prefill_flops(cfg, T)
            # frac: the step's flops over the matrix cores' peak; hbm_frac: the weights, which every step reads once,
            # over the memory's peak (what bounds a prompt of a few hundred tokens)
            prefills[T] = {"value": round(T / (ms / 1e3), 1), "tokens": T, "ms": round(ms, 3),
                           "frac": round(fl / (ms / 1e3) / PEAK_FLOPS[short], 4),
                           "hbm_frac": round(weight_bytes / (ms / 1e3) / 1e9 / PEAK_HBM_GBS, 4)}
            del eng
            torch.cuda.empty_cache()
            print(f"[bench] prefill {prefills[T]}", file=sys.stderr, flush=True)
    prefill_keys = list(prefills)

    # ---- the headline: decode at the default batch
    lens = prompt_lengths(args.prompt_lens, args.batch, args.prompt)
    dt, ctx0, ctx1 = decode_run(lens, args.steps, args.warmup)
    ms_step = dt / args.steps * 1e3
    gpu_ms_step = decode_run.gpu_ms
    value = args.batch * args.steps / dt
    points, point_rooflines = {}, {}
    for b in [int(x) for x in args.points.split(",") if x]:
        psteps = args.point_steps or args.steps
        pdt, p0, p1 = decode_run(prompt_lengths(args.prompt_lens, b, args.prompt), psteps, args.warmup)
        points[f"decode_b{b}"] = round(b * psteps / pdt, 1)
        point_rooflines[f"decode_b{b}"] = dict(roofline(pdt, psteps, p0, p1), ms_per_step=round(pdt / psteps * 1e3, 4))
        print(f"[bench] decode_b{b}: {points[f'decode_b{b}']} tok/s, {point_rooflines[f'decode_b{b}']}", file=sys.stderr, flush=True)

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
        "roofline": roofline(dt, args.steps, ctx0, ctx1),
        "points": points,
        "point_rooflines": point_rooflines,
    }
    for T in prefill_keys[1:]:
        line[f"prefill_{T}"] = prefills[T]
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
