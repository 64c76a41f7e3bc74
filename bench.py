"""Decode and prefill throughput of the Gemma 2 2B shape with random weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of a batch of 8 sequences that were prefilled with 2,048-token prompts;
by default the timed steps run the context from 2,048 out to 4,096.  The printed line also holds the
prefill of one 2,048-token prompt, the decode step's memory roofline (at the mean context of the timed
steps), and decode throughput at batch 1 and 64 over the same range.
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
    """Bytes a decode step has to read: every weight once, and the keys and values of the live requests."""
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
        pairs = sum(min(p + 1, w) if w else p + 1 for p in range(T))
        attn += 4 * cfg.num_attention_heads * cfg.head_dim * pairs
    return cfg.num_hidden_layers * per_layer + attn + 2 * n_logit_rows * H * cfg.vocab_size


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2048)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--preset", default="2b")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the preset (both numbers are reported)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64", help="other batch sizes to measure decode at ('' for none)")
    ap.add_argument("--point-steps", type=int, default=None, help="steps for the other batch sizes (default: --steps)")
    ap.add_argument("--no-prefill", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2

    import torch
    import alice_llm_amd as alice

    torch.cuda.set_device(0)
    raw = alice.preset(args.preset)
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    cfg = alice.config_from_dict(raw)
    t0 = time.time()
    model = alice.Model.random(cfg, seed=0, dtype=args.dtype, fast=True)
    print(f"[bench] model built in {time.time() - t0:.1f} s, weights {model.lm.weight_bytes() / 1e9:.2f} GB", file=sys.stderr, flush=True)
    elem = 2 if args.dtype == "bfloat16" else 4
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    gen = torch.Generator().manual_seed(0)

    def prompts(n):
        return [torch.randint(0, cfg.vocab_size, (args.prompt,), generator=gen).tolist() for _ in range(n)]

    def sync():
        torch.cuda.synchronize()

    def decode_run(batch, steps, warmup):
        """Prefill `batch` prompts, then time `steps` decode steps (greedy, tokens fed back)."""
        from alice_llm_amd.hip import ops
        per_seq = -(-(args.prompt + warmup + steps) // 64) * 64
        eng = model.engine(max_tokens=batch * max(args.context, per_seq), max_seqs=batch)
        slots = eng.open(batch)
        ps = prompts(batch)
        chunk = max(1, 16384 // args.prompt)                 # prefill a few sequences at a time
        ids = []
        for i in range(0, batch, chunk):
            logits = eng.step(slots[i:i + chunk], ps[i:i + chunk], "last")
            ids += ops.argmax(logits).tolist()
            print(f"[bench] prefilled {min(batch, i + chunk)}/{batch}", file=sys.stderr, flush=True)
        for _ in range(warmup):
            ids = ops.argmax(eng.step(slots, [[t] for t in ids], "last")).tolist()
        ctx0 = eng.length(slots[0])
        sync()
        t = time.perf_counter()
        for _ in range(steps):
            ids = ops.argmax(eng.step(slots, [[t_] for t_ in ids], "last")).tolist()
        sync()
        dt = time.perf_counter() - t
        ctx1 = eng.length(slots[0])
        eng.close(slots)
        del eng
        torch.cuda.empty_cache()
        return dt, ctx0, ctx1

    # ---- prefill of one 2,048-token prompt
    prefill = None
    if not args.no_prefill:
        eng = model.engine(max_tokens=args.context, max_seqs=1)
        p = prompts(1)
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
        fl = prefill_flops(cfg, args.prompt)
        prefill = {"value": round(args.prompt / (ms / 1e3), 1), "tokens": args.prompt, "ms": round(ms, 3),
                   "frac": round(fl / (ms / 1e3) / PEAK_FLOPS[short], 4)}
        del eng
        print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ---- the headline: decode at the default batch
    dt, ctx0, ctx1 = decode_run(args.batch, args.steps, args.warmup)
    ms_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    mid = (ctx0 + ctx1) // 2
    nbytes = decode_bytes(cfg, model.lm.weight_bytes(), [mid] * args.batch, elem)
    achieved = nbytes / (ms_step / 1e3) / 1e9
    points = {}
    for b in [int(x) for x in args.points.split(",") if x]:
        psteps = args.point_steps or args.steps
        pdt, _, _ = decode_run(b, psteps, args.warmup)
        points[f"decode_b{b}"] = round(b * psteps / pdt, 1)
        print(f"[bench] decode_b{b}: {points[f'decode_b{b}']} tok/s", file=sys.stderr, flush=True)

    line = {
        "metric": (f"decode tok/s @ batch {args.batch}, Gemma-2-{args.preset.upper()} {short} "
                   f"(points: batch {'/'.join(str(int(x)) for x in args.points.split(',') if x) or '-'}; "
                   f"prefill tok/s @ {args.prompt:,} tok)"),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic (uniform random token ids, random weights N(0, 0.02))",
        "config": {"model": f"gemma2-{args.preset}", "global_batch": args.batch, "seq_len": args.context,
                   "prompt_len": args.prompt, "context_start": ctx0, "context_end": ctx1, "parallelism": "single-gpu",
                   "layers": cfg.num_hidden_layers, "layers_of_model": full_layers, "hidden": cfg.hidden_size,
                   "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "sliding_window": cfg.sliding_window,
                   "weights_gb": round(model.lm.weight_bytes() / 1e9, 3)},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
