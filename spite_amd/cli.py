"""Command line in the manner of the reference's ``spite run``
(crates/spite-cli/src/main.rs:282-306, 498-562): ``-m/--model``, ``-p/--prompt``,
``--max-tokens`` (512), ``--temperature`` (1.0, 0 = greedy), ``--ctx``.  The engine works on
token ids; a text prompt needs a ``tokenizer.json`` in the model folder, otherwise give
``--prompt-ids`` or ``--prompt-len``.  Sampling defaults follow the reference's generate()
(crates/spite-executor/src/lib.rs:144-151, crates/spite-sampling/src/lib.rs:97-111): top-p
0.95, repetition penalty 1.1 over the last 64 tokens when the temperature is above zero, the
fixed seed of crates/spite-cli/src/main.rs:606.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

REFERENCE_SEED = 0x1234_5678_9ABC_DEF0


def _add_engine_args(ap):
    ap.add_argument("-m", "--model", default=os.environ.get("SPITE_MODEL"),
                    help="model folder (config.json, model.safetensors) [$SPITE_MODEL]")
    ap.add_argument("--config", help="config.json to build a model from with --random-weights")
    ap.add_argument("--random-weights", action="store_true", help="draw the weights from --seed instead of loading")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "bfloat16", "fp32", "float32"])
    ap.add_argument("--ctx", type=int, default=None, help="context window; default: the model's own maximum")
    ap.add_argument("--page-size", type=int, default=64)
    ap.add_argument("--num-pages", type=int, default=None, help="pages of every cache group (default: from --ctx)")
    ap.add_argument("--max-batch-tokens", type=int, default=2048)
    ap.add_argument("--max-requests", type=int, default=8)
    ap.add_argument("--seed", type=lambda s: int(s, 0), default=REFERENCE_SEED)


def _engine(args, n_requests=1):
    from .engine.engine import Engine
    source = args.model if not args.random_weights else (args.config or args.model)
    if source is None:
        raise SystemExit("spite: give --model DIR (or --config FILE --random-weights)")
    ctx = args.ctx or 4096
    t0 = time.time()
    eng = Engine(source, dtype=args.dtype, page_size=args.page_size, num_pages=args.num_pages,
                 cache_tokens=max(n_requests, 1) * (ctx + args.page_size), max_batch_tokens=args.max_batch_tokens,
                 max_requests=max(args.max_requests, n_requests), random_weights=args.random_weights, seed=args.seed)
    print(f"load time    : {time.time() - t0:.2f} s", file=sys.stderr)
    return eng


def _tokenizer(folder):
    path = os.path.join(folder or "", "tokenizer.json")
    if not os.path.exists(path):
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)


def cmd_run(args) -> int:
    import numpy as np
    tok = _tokenizer(args.model)
    if args.prompt_ids:
        prompts = [[int(x) for x in p.split(",") if x.strip()] for p in args.prompt_ids]
    elif args.prompt_len:
        prompts = None
    elif args.prompt is not None:
        if tok is None:
            raise SystemExit("spite run: -p needs tokenizer.json in the model folder; give --prompt-ids or --prompt-len")
        prompts = [tok.encode(args.prompt).ids]
    else:
        raise SystemExit("spite run: give -p TEXT, --prompt-ids or --prompt-len")
    eng = _engine(args, len(prompts) if prompts else 1)
    if prompts is None:
        rng = np.random.RandomState(args.seed % (1 << 32))
        prompts = [rng.randint(0, eng.spec.vocab_size, size=args.prompt_len).tolist()]
    arch = eng.spec.architecture
    print(f"engine       : spite_amd on gfx950, {arch}, {args.dtype}")
    if args.ctx:
        print(f"context      : {args.ctx} tokens")
    print(f"\nprompt       : {args.prompt if args.prompt is not None else prompts[0][:16]}")
    print(f"max tokens   : {args.max_tokens}")
    print(f"temperature  : {args.temperature}")
    sampling = dict(top_k=args.top_k, top_p=args.top_p, min_p=args.min_p,
                    repetition_penalty=(args.repetition_penalty if args.repetition_penalty is not None
                                        else (1.1 if args.temperature > 0 else 1.0)),
                    repeat_last_n=args.repeat_last_n)
    t0 = time.time()
    outs = eng.generate(prompts, max_tokens=args.max_tokens, temperature=args.temperature, seed=args.seed,
                        max_context=args.ctx, stop_token_ids=args.stop_token_ids or (), **sampling)
    secs = time.time() - t0
    n_prompt, n_new = sum(len(p) for p in prompts), sum(len(o) for o in outs)
    print(f"generate     : {n_prompt} prompt + {n_new} new tokens in {secs:.2f} s "
          f"({(n_prompt + n_new) / max(secs, 1e-9):.2f} tok/s)", file=sys.stderr)
    for o in outs:
        print("\n" + (tok.decode(o) if tok is not None and not args.ids_only else " ".join(str(t) for t in o)))
    return 0


def cmd_random_model(args) -> int:
    from .weights.random_init import write_random_model
    with open(args.config, "r", encoding="utf-8") as fh:
        cfg = json.load(fh)
    import torch
    # the same numbers either way; a GPU draws them sooner
    write_random_model(args.out, cfg, args.seed, args.std, args.dtype,
                       device="cuda:0" if torch.cuda.is_available() else None)
    print(f"wrote {args.out}/config.json and model.safetensors (seed {args.seed}, std {args.std})")
    return 0


def cmd_replay(args) -> int:
    import subprocess
    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    return subprocess.call([sys.executable, os.path.join(here, "bin", "trace_run"), *args.rest])


def cmd_bench(args) -> int:
    import subprocess
    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    return subprocess.call([sys.executable, os.path.join(here, "bench.py"), *args.rest])


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="spite", description="Llama 4 inference engine for one MI355X")
    sub = ap.add_subparsers(dest="cmd", required=True)
    run = sub.add_parser("run", help="generate tokens from a single prompt and print the output")
    _add_engine_args(run)
    run.add_argument("-p", "--prompt", help="prompt text (needs tokenizer.json)")
    run.add_argument("--prompt-ids", action="append", help="prompt as token ids, comma separated; may repeat")
    run.add_argument("--prompt-len", type=int, help="a random prompt of this many tokens")
    run.add_argument("--max-tokens", type=int, default=512, help="maximum tokens to generate")
    run.add_argument("--temperature", type=float, default=1.0, help="0 = greedy (deterministic), 1 = default")
    run.add_argument("--top-k", type=int, default=0)
    run.add_argument("--top-p", type=float, default=0.95)
    run.add_argument("--min-p", type=float, default=0.0)
    run.add_argument("--repetition-penalty", type=float, default=None,
                     help="default: 1.1 when the temperature is above zero, else off")
    run.add_argument("--repeat-last-n", type=int, default=64)
    run.add_argument("--stop-token-ids", type=lambda s: [int(x) for x in s.split(",")], default=None)
    run.add_argument("--ids-only", action="store_true", help="print token ids even when a tokenizer is there")
    run.set_defaults(fn=cmd_run)
    rm = sub.add_parser("random-model", help="write a model folder with random weights from a config and a seed")
    rm.add_argument("--config", required=True)
    rm.add_argument("--out", required=True)
    rm.add_argument("--seed", type=int, default=0)
    rm.add_argument("--std", type=float, default=0.02)
    rm.add_argument("--dtype", default=None, choices=["float32", "bfloat16", "float16"])
    rm.set_defaults(fn=cmd_random_model)
    rp = sub.add_parser("replay", help="trace replay (bin/trace_run)")
    rp.add_argument("rest", nargs=argparse.REMAINDER)
    rp.set_defaults(fn=cmd_replay)
    be = sub.add_parser("bench", help="the measurement of bench.py")
    be.add_argument("rest", nargs=argparse.REMAINDER)
    be.set_defaults(fn=cmd_bench)
    args = ap.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
