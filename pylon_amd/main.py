"""The command line.  The reference's ``main.py`` takes no arguments, refuses to start
without a GPU, and serves HTTP with every knob in a ``PYLON_*`` environment variable
(/root/reference/src/pylon/main.py:13-16; /root/reference/src/pylon/config.py:87-112).
This engine has no server; the same knobs are options here (the environment variables
still work as defaults), and the commands run on token ids:

    python main.py generate --model DIR --prompt-ids 1,2,3 [--prompt-ids ...]
    python main.py generate --random config.json --seed 0 --prompt-ids 1,2,3
    python main.py random-model --config config.json --seed 0 --out DIR
    python main.py replay --model DIR --dtype float32 --out DIR --max-tokens N  < steps.jsonl
    python main.py bench [bench.py's options]
    python main.py selftest
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def _add_serving_options(p: argparse.ArgumentParser) -> None:
    p.add_argument("--model", help="model folder (config.json, model.safetensors); PYLON_MODEL_PATH")
    p.add_argument("--dtype", choices=("bfloat16", "float32"))
    p.add_argument("--prefill-chunk-size", type=int)
    p.add_argument("--max-batch-size", type=int)
    p.add_argument("--max-queue-size", type=int)
    p.add_argument("--batch-wait-ms", type=float)
    p.add_argument("--max-gpu-utilization", type=float)
    p.add_argument("--weight-headroom-ratio", type=float)
    p.add_argument("--kv-cache-headroom-ratio", type=float)
    p.add_argument("--admit-skip", type=int)
    p.add_argument("--page-size", type=int)
    p.add_argument("--num-pages", type=int)
    p.add_argument("--cuda-graphs", action="store_true", default=None,
                   help="replay decode-only steps from HIP graphs")
    p.add_argument("--cuda-graph-max-tokens", type=int,
                   help="capture at start-up the graphs of requests of up to this many tokens")
    p.add_argument("--no-run-ahead", dest="run_ahead", action="store_false", default=None,
                   help="read every step's tokens before the next step is queued")


def _parse_ids(text: str):
    return [int(part) for part in text.replace(" ", "").split(",") if part]


def _generate(args) -> int:
    import torch

    if not torch.cuda.is_available():
        print("A GPU is required.", file=sys.stderr)
        return 1
    from .config import get_config
    from .engine.engine import Engine
    from .sampling import Sampling

    config = get_config(
        model_path=args.model, dtype=args.dtype, prefill_chunk_size=args.prefill_chunk_size,
        max_batch_size=args.max_batch_size, max_queue_size=args.max_queue_size,
        batch_wait_ms=args.batch_wait_ms, max_gpu_utilization=args.max_gpu_utilization,
        weight_headroom_ratio=args.weight_headroom_ratio,
        kv_cache_headroom_ratio=args.kv_cache_headroom_ratio, admit_skip=args.admit_skip,
        page_size=args.page_size, num_pages=args.num_pages, cuda_graphs=args.cuda_graphs,
        cuda_graph_max_tokens=args.cuda_graph_max_tokens, run_ahead=args.run_ahead,
    )
    prompts = [_parse_ids(text) for text in args.prompt_ids or []]
    if args.prompt_file:
        prompts.extend(json.loads(Path(args.prompt_file).read_text()))
    if not prompts:
        print("no prompts: give --prompt-ids or --prompt-file", file=sys.stderr)
        return 2
    sampling = Sampling(max_new_tokens=args.max_new_tokens, temperature=args.temperature,
                        top_p=args.top_p, seed=args.seed)
    if args.random:
        if args.model:
            print("give --model or --random, not both", file=sys.stderr)
            return 2
        engine = Engine.from_random(json.loads(Path(args.random).read_text()), args.seed, config=config)
    else:
        engine = Engine(config)
    try:
        if args.eos_token_id:
            eos = _parse_ids(args.eos_token_id)
        elif args.model:
            from .config import read_stop_token_ids

            eos = read_stop_token_ids(args.model) or None
        else:
            eos = getattr(engine.runner.config, "eos_token_id", None)
        results = engine.generate(prompts, sampling, eos)
    finally:
        engine.close()
    for prompt, result in zip(prompts, results):
        print(json.dumps({
            "prompt_tokens": len(prompt),
            "output_ids": result.output_ids,
            "finish_reason": result.finish_reason,
            "prefill_seconds": round(result.prefill_seconds, 6),
            "decode_seconds": round(sum(result.inter_token_seconds), 6),
        }))
    return 0


def _random_model(args) -> int:
    from .weights import write_random_model

    config = json.loads(Path(args.config).read_text())
    folder = write_random_model(args.out, config, args.seed, dtype=args.store_dtype,
                                norm_jitter=args.norm_jitter)
    print(folder)
    return 0


def main(argv=None) -> None:
    parser = argparse.ArgumentParser(prog="pylon", description=__doc__.split("\n\n")[0])
    sub = parser.add_subparsers(dest="command", required=True)

    gen = sub.add_parser("generate", help="generate from prompts given as token ids")
    _add_serving_options(gen)
    gen.add_argument("--random", metavar="CONFIG.json",
                     help="instead of --model: random weights (drawn from --seed) of this configuration")
    gen.add_argument("--prompt-ids", action="append", help="comma-separated token ids; repeatable")
    gen.add_argument("--prompt-file", help="JSON file: a list of lists of token ids")
    gen.add_argument("--max-new-tokens", type=int, default=256)
    gen.add_argument("--temperature", type=float, default=0.2)
    gen.add_argument("--top-p", type=float, default=0.95)
    gen.add_argument("--seed", type=int, default=0)
    gen.add_argument("--eos-token-id", help="comma-separated stop ids (default: the model folder's)")

    rnd = sub.add_parser("random-model", help="write a model folder with random weights")
    rnd.add_argument("--config", required=True, help="a config.json naming the architecture and sizes")
    rnd.add_argument("--seed", type=int, default=0)
    rnd.add_argument("--out", required=True)
    rnd.add_argument("--store-dtype", choices=("bfloat16", "float32"), default="bfloat16")
    rnd.add_argument("--norm-jitter", type=float, default=0.0)

    rep = sub.add_parser("replay", help="feed given token ids step by step and write logits",
                         add_help=False)
    rep.add_argument("rest", nargs=argparse.REMAINDER)

    ben = sub.add_parser("bench", help="decode and prefill throughput at the Qwen3-4B shape (bench.py)",
                         add_help=False)
    ben.add_argument("rest", nargs=argparse.REMAINDER)

    sub.add_parser("selftest", help="run a tiny random model three ways that must agree (whole prompt against "
                                    "token by token, bfloat16 against float32, the engine against a step loop)")

    args = parser.parse_args(argv)
    if args.command == "selftest":
        from .selftest import run as selftest

        try:
            selftest()
        except RuntimeError as error:
            print(error, file=sys.stderr)
            sys.exit(1)
        code = 0
    elif args.command == "generate":
        code = _generate(args)
    elif args.command == "random-model":
        code = _random_model(args)
    elif args.command == "bench":
        import runpy

        script = Path(__file__).resolve().parent.parent / "bench.py"
        sys.argv = [str(script), *args.rest]
        runpy.run_path(str(script), run_name="__main__")
        code = 0
    else:
        from .engine.replay import main as replay_main

        code = replay_main(args.rest)
    raise SystemExit(code)


if __name__ == "__main__":
    main()
