"""Command line.

    python -m lite_llama_amd generate --model DIR --prompt-ids 1,2,3 [--prompt-ids 4,5] [--max-new-tokens N]
                                      [--dtype bfloat16|float32] [--temperature T --top-p P --repetition-penalty R]
    python -m lite_llama_amd trace    --model DIR --dtype ... --out DIR --max-tokens N      (= bin/trace_run)
    python -m lite_llama_amd build    [--part NAME] [--force]

``generate`` works on token ids (no tokenizer ships with the engine): layered models (config.json ``architecture``) run through
the continuous-batching engine over ragged steps, llama-shaped checkpoints (``model_type``) through the padded-prefill /
captured-decode engine.  One JSON line per prompt: ``{"prompt": [...], "generated": [...]}``.
"""

from __future__ import annotations

import argparse
import json
import os
import sys


def _generate(args) -> int:
    import torch

    from . import _lib
    from .weights import MODEL_FAMILIES, load_pretrained, model_family

    with open(os.path.join(args.model, "config.json")) as f:
        config = json.load(f)
    prompts = [[int(t) for t in p.replace(" ", "").split(",") if t] for p in args.prompt_ids]
    layered = model_family(config) in MODEL_FAMILIES
    if layered:
        _lib.use_part("ragged")
    if not torch.cuda.is_available():
        print("generate: no GPU (there is no CPU path)", file=sys.stderr)
        return 2
    if layered:
        from .engine import GenerationEngine, SamplingParams

        dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
        model = load_pretrained(args.model, device="cuda", dtype=dtype)
        params = SamplingParams(max_new_tokens=args.max_new_tokens, temperature=args.temperature, top_p=args.top_p,
                                repetition_penalty=args.repetition_penalty, eos_token_id=args.eos_token_id)
        page = args.page_size
        pool = args.max_tokens or sum(-(-(len(p) + args.max_new_tokens) // page) * page for p in prompts[:args.max_requests])
        engine = GenerationEngine(model, pool, max_requests=args.max_requests, block_size=page,
                                  max_step_tokens=args.max_step_tokens, seed=args.seed, capture_decode=args.capture_decode)
        outs = engine.generate(prompts, params)
    else:
        import types

        from .executor import DecodeEngine

        model = load_pretrained(args.model, device="cuda", quantization=args.quantization)
        longest = max(len(p) for p in prompts)
        ids = torch.zeros(len(prompts), longest, dtype=torch.long, device="cuda")
        for i, p in enumerate(prompts):
            ids[i, :len(p)] = torch.tensor(p)
        lens = torch.tensor([len(p) for p in prompts], dtype=torch.int32, device="cuda")
        sampling = None
        if args.temperature != 0.0 or args.repetition_penalty != 1.0:
            sampling = types.SimpleNamespace(temperature=args.temperature, top_p=args.top_p,
                                             repetition_penalty=args.repetition_penalty)
        eng = DecodeEngine(model, max_batch=len(prompts), max_seq_len=longest + args.max_new_tokens + 1, device="cuda")
        first = eng.prefill(ids, lens, sampling=sampling)
        rest = eng.decode(first, args.max_new_tokens - 1, sampling=sampling) if args.max_new_tokens > 1 else None
        outs = [[int(first[i])] + ([int(t) for t in rest[i]] if rest is not None else []) for i in range(len(prompts))]
    for p, o in zip(prompts, outs):
        print(json.dumps({"prompt": p, "generated": o}))
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m lite_llama_amd", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate")
    g.add_argument("--model", required=True)
    g.add_argument("--prompt-ids", action="append", required=True, help="comma-separated token ids; repeat for a batch")
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--repetition-penalty", type=float, default=1.0)
    g.add_argument("--eos-token-id", type=int, default=None)
    g.add_argument("--quantization", default=None, help="load-time quantisation scheme (llama-shaped checkpoints)")
    g.add_argument("--max-tokens", type=int, default=0, help="cache pool in tokens (default: what the first requests need)")
    g.add_argument("--max-requests", type=int, default=4)
    g.add_argument("--max-step-tokens", type=int, default=512)
    g.add_argument("--page-size", type=int, default=64)
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--capture-decode", action="store_true", help="layered models: replay decode-only steps from hipGraphs")
    sub.add_parser("trace", add_help=False)
    b = sub.add_parser("build")
    b.add_argument("--part", default=None)
    b.add_argument("--force", action="store_true")
    args, rest = ap.parse_known_args(argv)
    if args.cmd == "trace":
        from .trace_replay import main as trace_main

        return trace_main(rest)
    if rest:
        ap.error(f"unrecognised arguments: {' '.join(rest)}")
    if args.cmd == "build":
        from . import build

        print(build.build(force=args.force, part=args.part))
        return 0
    return _generate(args)


if __name__ == "__main__":
    sys.exit(main())
