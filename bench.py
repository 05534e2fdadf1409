"""Decode and prefill throughput of the engine at the Qwen3-4B shape, with random weights
and uniform-random token ids, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]
                    [--shape 4b|8b|32b] [--prompt-len N]

Everything goes the product's own way.  Start-up is ``Runner.from_random``: the fit check,
the measured activation headroom, the page pool sized from the card's memory and the decode
graphs captured before serving, as ``main.py generate --random`` does it.  Requests go through
``Engine``: queue, admission, prompts cut into portions of at most 2,048 tokens, ticks.

A "step" is one tick of the engine once all ``batch`` requests decode: one token for each of
them through the step function (replayed from a HIP graph), greedy sampling on the device, and
the read of the chosen ids by the host; as in serving, a tick queues its step before it reads
the ids of the step before (they are fed back on the device).  ``value`` is decoded tokens per
second at the default batch of 8.  The same line carries the prefill of 2,048 tokens (one
request from its arrival to its first token), the decode step's share of the HBM roofline, and
under ``points`` decode rates at batch 1 and 64, with the reference's default sampling options
instead of greedy, at contexts of 2,000, 4,096 and 8,000 tokens, a prompt
of 8,191 tokens in four portions, a step of 64 decoded tokens beside a 2,048-token portion, and
two rates over whole requests (queueing, admission and prefill included): ``engine_b8`` with the
same 128-token prompts and 512 new tokens, ``engine_prefill_heavy_b8`` with 2,048-token prompts
and 32 new tokens.  ``--shape`` and ``--prompt-len`` measure the same at the Qwen3-8B and 32B
layer sizes and at longer contexts.
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

# MI355X published peaks.
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

# The benchmark configuration: Qwen3-4B shape.
SHAPE_4B = dict(
    num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
    head_dim=128, intermediate_size=9728, vocab_size=151936, rope_theta=5000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=8192,
)
SHAPE_8B = dict(
    num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
    head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=32768,
)
SHAPE_32B = dict(
    num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
    head_dim=128, intermediate_size=25600, vocab_size=151936, rope_theta=1000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=32768,
)
SHAPES = {"4b": SHAPE_4B, "8b": SHAPE_8B, "32b": SHAPE_32B}
PAGE_SIZE = 256
PROMPT_LEN = 128
NEW_TOKENS = 512
PREFILL_TOKENS = 2048
MOST_NEW_TOKENS = 2048  # what a request may ask for (Sampling's range, the reference's)
# The reference's own published figure for this workload (128-token prompts, 512 new tokens,
# 8 requests at a time, Qwen3-4B): 199.8 output tokens/s, through its server on one NVIDIA L4
# (/root/reference/README.md:73).  Other hardware: the ratio says how far apart the two
# set-ups are, not how the engines compare on one card.
REFERENCE_DECODE_B8 = 199.8


def config_json(shape: dict, layers: int) -> dict:
    cfg = dict(shape, num_hidden_layers=layers)
    cfg.update(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu")
    return cfg


def serving_config(dtype: str, max_batch: int, graphs: bool, **more):
    from pylon_amd.config import PylonConfig

    return PylonConfig(dtype=dtype, max_batch_size=max_batch, max_queue_size=max(max_batch, 1), page_size=PAGE_SIZE,
                       prefill_chunk_size=PREFILL_TOKENS, cuda_graphs=graphs, **more)


def weight_bytes(runner) -> int:
    """Bytes of every weight a decode step reads once: all layer matrices and vectors and
    the vocabulary head (the embedding table itself is only gathered from)."""
    total = 0
    for path, owner, name in runner.model.named_params():
        if path == "embed" and not runner.model.spec.tie_word_embeddings:
            continue
        t = owner.params[name]
        total += t.numel() * t.element_size()
    return total


def linear_flops_per_token(cfg) -> float:
    q = cfg.num_attention_heads * cfg.head_dim
    kv = cfg.num_key_value_heads * cfg.head_dim
    per_layer = cfg.hidden_size * (q + 2 * kv) + q * cfg.hidden_size + 3 * cfg.hidden_size * cfg.intermediate_size
    return 2.0 * cfg.num_hidden_layers * per_layer


def attention_flops(cfg, new_tokens: int, cached: int = 0) -> float:
    """Score and value products of ``new_tokens`` tokens that follow ``cached`` ones (causal)."""
    pairs = new_tokens * cached + new_tokens * (new_tokens + 1) / 2
    return 4.0 * cfg.num_hidden_layers * cfg.num_attention_heads * cfg.head_dim * pairs


class Serving:
    """``batch`` requests of ``prompt_len`` random ids each, brought through the engine to the
    point where every one of them decodes; then ticks can be timed."""

    def __init__(self, runner, cfg, args, batch: int, prompt_len: int, ticks: int, seed: int, room: int = 0,
                 temperature: float = 0.0, top_p: float = 1.0):
        import numpy as np

        from pylon_amd.engine.engine import Engine
        from pylon_amd.sampling import Sampling

        self.runner, self.cfg, self.batch = runner, cfg, batch
        self.rng = np.random.default_rng(seed)
        config = serving_config(args.dtype, batch + room, runner.graphs is not None)
        self.engine = Engine(config, runner=runner)
        # the prompts' portions take ticks in which the first requests already decode
        prefill_ticks = -(-batch * prompt_len // PREFILL_TOKENS) + 2
        limit = runner.model.spec.max_positions - prompt_len
        self.new_tokens = min(MOST_NEW_TOKENS, limit, ticks + prefill_ticks + 8)
        self.ticks = self.new_tokens - prefill_ticks - 8
        if self.ticks < 1:
            raise SystemExit(f"bench.py: {prompt_len}-token prompts leave no room for decode steps")
        sampling = Sampling(max_new_tokens=self.new_tokens, temperature=temperature, top_p=top_p, seed=seed)
        self.futures = [self.engine.enqueue(self.rng.integers(0, cfg.vocab_size, prompt_len).tolist(), None, sampling)
                        for _ in range(batch)]
        while True:
            self.engine.tick()
            decoding, portions = self.engine.last_step
            if len(decoding) == batch and not portions:
                break

    def timed_ticks(self, count: int, warmup: int):
        """(seconds, mean cached tokens read per step over all rows) of ``count`` ticks."""
        import torch

        if warmup + count > self.ticks:
            raise SystemExit(f"bench.py: {warmup} + {count} steps do not fit the requests' {self.ticks} decode ticks")
        for _ in range(warmup):
            self.engine.tick()
        self.ticks -= warmup + count
        seqs = self.runner.manager.live_sequences()
        torch.cuda.synchronize()
        context = 0
        started = time.perf_counter()
        for _ in range(count):
            context += sum(s.length + 1 for s in seqs)
            self.engine.tick()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        decoding, portions = self.engine.last_step
        assert len(decoding) == self.batch and not portions and self.engine.steps_run >= count
        return elapsed, context / count

    def mixed_tick_ms(self, repeats: int) -> float:
        """Milliseconds of device time of a step that carries every decoding request's token
        beside a PREFILL_TOKENS portion of a new prompt (median): events around the tick that
        queues it.  The engine must have been made with ``room=1``."""
        import torch

        from pylon_amd.sampling import Sampling

        times = []
        for _ in range(repeats + 1):
            prompt = self.rng.integers(0, self.cfg.vocab_size, PREFILL_TOKENS).tolist()
            future = self.engine.enqueue(prompt, None, Sampling(max_new_tokens=1, temperature=0.0))
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            self.engine.tick()
            end.record()
            decoding, portions = self.engine.last_step
            assert len(decoding) == self.batch and [count for _, count in portions] == [PREFILL_TOKENS]
            while not future.done():
                self.engine.tick()
            self.ticks -= 3
            end.synchronize()
            times.append(start.elapsed_time(end))
        times = sorted(times[1:])
        return times[len(times) // 2]

    def finish(self) -> None:
        self.engine.run_until_idle()
        results = [f.result(timeout=0) for f in self.futures]
        assert all(len(r.output_ids) == self.new_tokens for r in results)
        self.engine.close()


def decode_point(runner, cfg, args, batch: int, prompt_len: int, steps: int, seed: int, mixed: bool = False,
                 temperature: float = 0.0, top_p: float = 1.0) -> dict:
    """Tokens per second and roofline share of decode steps of ``batch`` requests at this context
    (greedy, or sampled with a temperature and top-p)."""
    serving = Serving(runner, cfg, args, batch, prompt_len, steps + args.warmup + (24 if mixed else 0), seed,
                      room=1 if mixed else 0, temperature=temperature, top_p=top_p)
    elapsed, context = serving.timed_ticks(steps, args.warmup)
    out = {"tokens_per_s": batch * steps / elapsed, "ms": 1e3 * elapsed / steps,
           "bytes": weight_bytes(runner) + context * runner.manager.bytes_per_token, "context": context / batch}
    out["frac"] = out["bytes"] / (elapsed / steps) / HBM_BYTES_PER_S
    if mixed:
        out["mixed_ms"] = serving.mixed_tick_ms(repeats=5)
    serving.finish()
    return out


def prefill_run(runner, cfg, args, tokens: int, repeats: int, seed: int) -> float:
    """Seconds from a request's arrival to its first token, for one prompt of ``tokens`` random
    ids and nothing else running (portions of at most PREFILL_TOKENS); the median."""
    import numpy as np
    import torch

    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    rng = np.random.default_rng(seed)
    engine = Engine(serving_config(args.dtype, 1, runner.graphs is not None), runner=runner)
    times = []
    for _ in range(repeats + 1):
        prompt = rng.integers(0, cfg.vocab_size, tokens).tolist()
        torch.cuda.synchronize()
        started = time.perf_counter()
        result, = engine.generate([prompt], Sampling(max_new_tokens=1, temperature=0.0))
        times.append(time.perf_counter() - started)
        assert len(result.output_ids) == 1
    engine.close()
    times = sorted(times[1:])  # the first run warms the library's kernels up
    return times[len(times) // 2]


def engine_run(runner, cfg, args, batch: int, seed: int, prompt_len: int = PROMPT_LEN, new_tokens: int = NEW_TOKENS):
    """Whole requests: ``batch`` requests of ``prompt_len`` random ids and ``new_tokens`` greedy
    tokens each, queued at once; generated tokens per second from the first request's arrival
    to the last one's end (admission, the prompts' prefill, ticks, sampling and the host's
    reading of every token included), and the median time from a request's arrival to its
    first token in milliseconds."""
    import numpy as np
    import torch

    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    rng = np.random.default_rng(seed)
    prompts = [rng.integers(0, cfg.vocab_size, prompt_len).tolist() for _ in range(batch)]
    engine = Engine(serving_config(args.dtype, batch, runner.graphs is not None), runner=runner)
    sampling = Sampling(max_new_tokens=new_tokens, temperature=0.0)
    torch.cuda.synchronize()
    started = time.perf_counter()
    results = engine.generate(prompts, sampling)
    elapsed = time.perf_counter() - started
    engine.close()
    assert all(len(r.output_ids) == new_tokens for r in results)
    first = sorted(r.first_token_seconds for r in results)
    return batch * new_tokens / elapsed, 1e3 * first[len(first) // 2]


def measured_peaks() -> dict:
    """What this very device reaches on the two resources the fractions are priced against:
    reading memory (this repository's streaming read kernel over 2 GiB, larger than every
    cache) and bfloat16 matrix products (the library's product of 8,192-sized squares)."""
    import torch

    from pylon_amd.kernels import ops

    data = torch.empty(1 << 29, dtype=torch.int32, device="cuda:0").fill_(1)
    sink = torch.zeros(1, dtype=torch.int32, device="cuda:0")

    def timed(fn, repeats):
        fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(repeats):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) * 1e-3 / repeats

    read = data.numel() * 4 / timed(lambda: ops.probe_read(data, sink), 10)
    del data
    a = torch.randn(8192, 8192, device="cuda:0", dtype=torch.bfloat16)
    b = torch.randn(8192, 8192, device="cuda:0", dtype=torch.bfloat16)
    flops = 2.0 * 8192 ** 3 / timed(lambda: torch.mm(a, b.t()), 10)
    return {"hbm_read_gbs": round(read / 1e9, 1), "bf16_gemm_tflops": round(flops / 1e12, 1)}


def main() -> int:
    parser = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=NEW_TOKENS)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--shape", choices=sorted(SHAPES), default="4b", help="layer sizes (default: Qwen3-4B)")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has")
    parser.add_argument("--prompt-len", type=int, default=PROMPT_LEN, help="tokens cached before decoding starts")
    parser.add_argument("--context-length", type=int, default=None,
                        help="longest request in tokens (default: the shape's max_position_embeddings)")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--temperature", type=float, default=0.0,
                        help="sample the timed run's tokens at this temperature (default 0: the largest logit)")
    parser.add_argument("--top-p", type=float, default=1.0, help="with --temperature: the nucleus kept")
    parser.add_argument("--no-graphs", action="store_true", help="launch decode steps kernel by kernel")
    parser.add_argument("--no-points", action="store_true", help="skip the other batch sizes and contexts")
    parser.add_argument("--no-prefill", action="store_true")
    parser.add_argument("--no-peaks", action="store_true", help="skip the probes of this device's own peaks")
    parser.add_argument("--mixed", action="store_true",
                        help="also time a step of --batch decoded tokens beside a 2,048-token prompt portion")
    parser.add_argument("--prefill-only", action="store_true",
                        help="only the prefill measurement (for profiling); prints its part of the record")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus must be 1")
        return 2
    import torch

    if not torch.cuda.is_available():
        print("bench.py: A GPU is required.", file=sys.stderr)
        return 1
    from pylon_amd.engine import Runner

    shape = dict(SHAPES[args.shape])
    if args.context_length:
        shape["max_position_embeddings"] = args.context_length
    layers = args.layers or shape["num_hidden_layers"]
    context_length = shape["max_position_embeddings"]
    prompt_len = args.prompt_len
    max_batch = args.batch + 1 if args.no_points else max(64, args.batch) + 1
    # The product's start-up: weights drawn in place, the pool sized from the card's memory
    # under the serving options (at most max_batch requests of the longest length), graphs.
    raw = config_json(shape, layers)
    runner = Runner.from_random(raw, 0, serving_config(args.dtype, max_batch, not args.no_graphs), std=0.02)
    cfg = runner.config
    dtype_key = "bf16" if args.dtype == "bfloat16" else "fp32"
    if args.prefill_only:
        seconds = prefill_run(runner, cfg, args, PREFILL_TOKENS, repeats=5, seed=2)
        print(json.dumps({"prefill": {"value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS,
                                      "ms": round(1e3 * seconds, 3)}}))
        return 0

    serving = Serving(runner, cfg, args, args.batch, prompt_len, args.steps + args.warmup + (24 if args.mixed else 0),
                      seed=1, room=1 if args.mixed else 0, temperature=args.temperature, top_p=args.top_p)
    steps = min(args.steps, serving.ticks - args.warmup - (24 if args.mixed else 0))
    elapsed, mean_context = serving.timed_ticks(steps, args.warmup)
    mixed_ms = serving.mixed_tick_ms(repeats=5) if args.mixed else None
    serving.finish()
    ms_per_step = 1e3 * elapsed / steps
    value = args.batch * steps / elapsed
    step_bytes = weight_bytes(runner) + mean_context * runner.manager.bytes_per_token
    achieved = step_bytes / (elapsed / steps)

    headline = (args.shape == "4b" and args.batch == 8 and prompt_len == PROMPT_LEN and args.dtype == "bfloat16"
                and layers == shape["num_hidden_layers"] and args.temperature == 0)
    drawn = f", temperature {args.temperature:g}, top-p {args.top_p:g}" if args.temperature > 0 else ""
    record = {
        "metric": f"decode tokens/s, Qwen3-{args.shape.upper()} shape, batch {args.batch}, {prompt_len}-token prompts{drawn}",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / REFERENCE_DECODE_B8, 2) if headline else None, "dtype": dtype_key, "data": "synthetic",
        "config": {
            "model": f"qwen3-{args.shape}-shape-random", "layers": layers,
            "layers_full": shape["num_hidden_layers"], "hidden": cfg.hidden_size,
            "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "global_batch": args.batch, "seq_len": prompt_len, "new_tokens": steps,
            "context_length": context_length, "page_size": PAGE_SIZE, "prefill_tokens": PREFILL_TOKENS,
            "hip_graphs": runner.graphs is not None, "pool_pages": runner.manager.num_pages,
            "startup_s": round(runner.startup["total_s"], 2), "parallelism": "single-gpu",
            "baseline": "reference on one NVIDIA L4, 8 clients: 199.8 tokens/s",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_BYTES_PER_S / 1e9,
                     "unit": "GB/s", "frac": round(achieved / HBM_BYTES_PER_S, 4)},
        "startup": {k: round(v, 2) for k, v in runner.startup.items()},
    }
    if runner.graphs is not None:
        record["startup"]["graphs"] = len(runner.graphs.captured)
    if not args.no_prefill:
        seconds = prefill_run(runner, cfg, args, PREFILL_TOKENS, repeats=5, seed=2)
        flops = (linear_flops_per_token(cfg) * PREFILL_TOKENS + attention_flops(cfg, PREFILL_TOKENS)
                 + 2.0 * cfg.hidden_size * cfg.vocab_size)
        record["prefill"] = {"value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS,
                             "ms": round(1e3 * seconds, 3),
                             "frac": round(flops / seconds / PEAK_FLOPS[dtype_key], 4)}
    if not args.no_peaks:
        peaks = measured_peaks()
        record["measured_peaks"] = peaks
        record["roofline"]["frac_of_measured"] = round(achieved / 1e9 / peaks["hbm_read_gbs"], 4)
        if "prefill" in record and dtype_key == "bf16":
            record["prefill"]["frac_of_measured"] = round(
                record["prefill"]["frac"] * PEAK_FLOPS[dtype_key] / 1e12 / peaks["bf16_gemm_tflops"], 4)
    if mixed_ms is not None:
        record["mixed"] = {"decodes": args.batch, "chunk": PREFILL_TOKENS, "ms": round(mixed_ms, 3)}
    if not args.no_points:
        points = {}
        few = max(32, min(steps, 256))

        def put(name, point):
            points[name] = round(point["tokens_per_s"], 1)
            points[name + "_hbm_frac"] = round(point["frac"], 4)

        put("decode_b1", decode_point(runner, cfg, args, 1, prompt_len, few, seed=4))
        put("decode_b64", decode_point(runner, cfg, args, 64, prompt_len, few, seed=67))
        # the reference's default sampling options (/root/reference/src/pylon/api/types.py:6-9)
        # instead of greedy: one workgroup per row norms, cuts at top-p and draws
        put("decode_b8_sampled", decode_point(runner, cfg, args, 8, prompt_len, few, seed=68, temperature=0.2,
                                              top_p=0.95))
        if headline:
            # longer contexts: the decode attention's share grows, its keys are cut over workgroups
            put("decode_b8_ctx2000", decode_point(runner, cfg, args, 8, 2000, 48, seed=15))
            put("decode_b8_ctx4096", decode_point(runner, cfg, args, 8, 4096, 64, seed=11))
            put("decode_b1_ctx8000", decode_point(runner, cfg, args, 1, 8000, 64, seed=12))
            point = decode_point(runner, cfg, args, 64, 4096, 64, seed=13, mixed=True)
            put("decode_b64_ctx4096", point)
            # a step of 64 decoded tokens (about 4,200 cached each) beside a 2,048-token portion
            chunk_flops = (linear_flops_per_token(cfg) * (PREFILL_TOKENS + 64) + attention_flops(cfg, PREFILL_TOKENS)
                           + 65 * 2.0 * cfg.hidden_size * cfg.vocab_size)
            points["mixed_b64_chunk2048_ms"] = round(point["mixed_ms"], 3)
            points["mixed_b64_chunk2048_hbm_frac"] = round(point["bytes"] / (point["mixed_ms"] * 1e-3) / HBM_BYTES_PER_S, 4)
            points["mixed_b64_chunk2048_flops_frac"] = round(chunk_flops / (point["mixed_ms"] * 1e-3) / PEAK_FLOPS[dtype_key], 4)
            # one prompt as long as the context allows (8,191 tokens: 8,192 less the token it produces), in portions
            long_prompt = context_length - 1
            seconds = prefill_run(runner, cfg, args, long_prompt, repeats=3, seed=14)
            flops = linear_flops_per_token(cfg) * long_prompt + attention_flops(cfg, long_prompt)
            points[f"prefill_{long_prompt}"] = round(long_prompt / seconds, 1)
            points[f"prefill_{long_prompt}_flops_frac"] = round(flops / seconds / PEAK_FLOPS[dtype_key], 4)
        rate, first_ms = engine_run(runner, cfg, args, batch=8, seed=9, prompt_len=prompt_len)
        points["engine_b8"], points["engine_b8_first_token_ms"] = round(rate, 1), round(first_ms, 2)
        # the reference's other published workload: 2,048-token prompts, 32 new tokens, 8 at a time
        # (53.7 output tokens/s and 847 ms to the first token on its L4, /root/reference/README.md:76,90)
        rate, first_ms = engine_run(runner, cfg, args, batch=8, seed=10, prompt_len=PREFILL_TOKENS, new_tokens=32)
        points["engine_prefill_heavy_b8"] = round(rate, 1)
        points["engine_prefill_heavy_b8_first_token_ms"] = round(first_ms, 2)
        record["points"] = points
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
