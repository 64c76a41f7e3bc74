"""Command line: python -m alice_llm_amd.generate --model DIR --prompt-ids 2,651,9456 --max-tokens 32

Option names and meanings follow the reference's generate examples where it has them
(--model, --max-tokens default 256, --temperature, --top-k: examples/elyza_gguf.rs:81-117 and
examples/generate_gpu.rs:31-40; temperature 0 is greedy, generate_gpu.rs:122; --logits-dump N writes,
for every request, the top-5 logits of its first N generated positions as JSON lines to stderr while the
request runs: the logits of the run's own steps and the token its sampler drew from them,
examples/elyza_gguf.rs:31-76, 200-259; --dump-logits FILE sends the same lines to a file instead, for
every generated position unless --logits-dump N limits them).  There is no tokenizer here: prompts are token ids, and so is the
output.  The closing lines are the reference's (examples/elyza_gguf.rs:277-286).
"""
from __future__ import annotations

import argparse
import json
import sys
from typing import List


def _ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m alice_llm_amd.generate", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", help="folder with config.json and model.safetensors")
    ap.add_argument("--random-weights", action="store_true", help="random weights from --preset/--config and --weights-seed")
    ap.add_argument("--preset", help="a named configuration (with --random-weights)")
    ap.add_argument("--config", help="a config.json file (with --random-weights)")
    ap.add_argument("--weights-seed", type=int, default=0)
    ap.add_argument("--prompt-ids", action="append", default=[], help="token ids '1,2,3'; repeat for a batch")
    ap.add_argument("--prompt-file", action="append", default=[], help="file with one prompt's token ids per line")
    ap.add_argument("--max-tokens", type=int, default=256, help="cap on new tokens per sequence")
    ap.add_argument("--temperature", type=float, default=0.0, help="0 is greedy")
    ap.add_argument("--top-k", type=int, default=0, help="keep the k most likely tokens (0: off)")
    ap.add_argument("--top-p", type=float, default=1.0, help="nucleus mass (1: off)")
    ap.add_argument("--seed", type=int, default=0, help="sampler seed")
    ap.add_argument("--stop-ids", default=None, help="stop token ids '1,107' (default: the configuration's eos)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32", "bf16", "fp32"], default=None)
    ap.add_argument("--max-batch", type=int, default=None, help="most sequences in one batch")
    ap.add_argument("--logits-dump", type=int, default=0,
                    help="dump the top-5 logits of each request's first N generated positions (JSON lines on stderr)")
    ap.add_argument("--dump-logits", metavar="FILE", default=None,
                    help="write the dump's JSON lines to FILE instead of stderr (every generated position, or the "
                         "first N with --logits-dump N)")
    ap.add_argument("--ignore-unexpected-tensors", action="store_true",
                    help="tensors in the folder that the model does not declare are warned about instead of refused")
    ap.add_argument("--keep-stored-dtype", action="store_true",
                    help="with --dtype bfloat16: matrices stored in float32 stay float32 instead of being rounded once at load")
    args = ap.parse_args(argv)

    import alice_llm_amd as alice

    prompts = [_ids(p) for p in args.prompt_ids]
    for path in args.prompt_file:
        with open(path) as f:
            prompts += [_ids(line) for line in f if line.strip()]
    if not prompts:
        ap.error("give at least one prompt with --prompt-ids or --prompt-file")
    if args.random_weights:
        if args.config:
            with open(args.config) as f:
                raw = json.load(f)
        elif args.preset:
            raw = alice.preset(args.preset)
        else:
            ap.error("--random-weights needs --preset or --config")
        print(f"Building random weights (seed {args.weights_seed})", flush=True)
        model = alice.load(raw, dtype=args.dtype, random_seed=args.weights_seed, keep_stored_dtype=args.keep_stored_dtype)
    else:
        if not args.model:
            ap.error("give --model DIR, or --random-weights with --preset/--config")
        print(f"Loading model: {args.model}", flush=True)
        model = alice.load(args.model, dtype=args.dtype, strict=not args.ignore_unexpected_tensors,
                           keep_stored_dtype=args.keep_stored_dtype)

    stop = _ids(args.stop_ids) if args.stop_ids is not None else None
    observer = dump_file = None
    if args.dump_logits:
        dump_file = open(args.dump_logits, "w")
        observer = _logits_dumper(args.logits_dump if args.logits_dump > 0 else None, dump_file)
    elif args.logits_dump > 0:
        observer = _logits_dumper(args.logits_dump, sys.stderr)
    try:
        results = model.generate(prompts, max_new_tokens=args.max_tokens, temperature=args.temperature,
                                 top_k=args.top_k, top_p=args.top_p, seed=args.seed, stop_token_ids=stop,
                                 max_batch=args.max_batch, observer=observer)
    finally:
        if dump_file is not None:
            dump_file.close()
    for i, r in enumerate(results):
        print(f"[{i}] " + ",".join(str(t) for t in r.tokens) + f"  ({r.finish_reason})")
    print("---")
    g = sum(r.tokens_generated for r in results)
    p = sum(r.prompt_tokens for r in results)
    seen, prefill, decode = set(), 0.0, 0.0
    for r in results:                       # times are per batch; count each batch once
        key = (r.prefill_ms, r.decode_ms)
        if key not in seen:
            seen.add(key)
            prefill += r.prefill_ms
            decode += r.decode_ms
    print(f"Tokens: {g} generated, {p} prompt")
    tps = g / (decode / 1e3) if decode > 0 else 0.0
    print(f"Speed: {tps:.1f} tok/s ({prefill:.0f} prefill + {decode:.0f} decode = {prefill + decode:.0f} total ms)")
    return 0


def _logits_dumper(n, out):
    """An observer of the generation loop: for each request's first n generated positions (n None: all of them)
    one JSON line to `out` with the request, the position the logits belong to, the token drawn there and the
    five largest logits."""
    import torch
    seen = {}

    def observe(requests, positions, logits, tokens) -> None:
        rows = [i for i, r in enumerate(requests) if n is None or seen.get(r, 0) < n]
        if not rows:
            return
        top = torch.topk(logits[rows], min(5, logits.shape[1]), dim=-1)
        values, indices = top.values.tolist(), top.indices.tolist()
        for j, i in enumerate(rows):
            r = requests[i]
            seen[r] = seen.get(r, 0) + 1
            print(json.dumps({"request": r, "position": positions[i], "token": int(tokens[i]),
                              "top5": [[int(t), float(v)] for t, v in zip(indices[j], values[j])]}),
                  file=out, flush=True)
    return observe


if __name__ == "__main__":
    sys.exit(main())
