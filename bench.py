"""Decode and prefill throughput of the engine at the Qwen3-4B shape, with random weights
and uniform-random token ids, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]
                    [--shape 4b|8b|32b] [--prompt-len N]

A "step" is one decode step: one token for each of ``batch`` running requests through
the step function, then greedy sampling on the device and the copy of the chosen ids to
the host.  As in the engine's ticks, a step is queued before the host has read the ids of
the step before it (they are fed back on the device), and every step's ids are read.  ``value`` is decoded tokens per second at the default batch of 8.  The same
line carries the prefill of 2,048 tokens, the decode step's share of the HBM roofline,
decode rates at batch 1 and 64, and two rates through the scheduler (queueing, admission and
the prompts' prefill included): ``points.engine_b8`` with the same 128-token prompts and 512
new tokens, ``points.engine_prefill_heavy_b8`` with 2,048-token prompts and 32 new tokens.
``--shape`` and ``--prompt-len`` measure the same at the Qwen3-8B and 32B layer sizes and
at longer contexts; the default run is the 4B shape with 128-token prompts.
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
# The reference's own published figure for this workload (128-token prompts, 512 new tokens,
# 8 requests at a time, Qwen3-4B): 199.8 output tokens/s, through its server on one NVIDIA L4
# (/root/reference/README.md:73).  Other hardware: the ratio says how far apart the two
# set-ups are, not how the engines compare on one card.
REFERENCE_DECODE_B8 = 199.8


def config_json(shape: dict, layers: int) -> dict:
    cfg = dict(shape, num_hidden_layers=layers)
    cfg.update(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu")
    return cfg


def build_runner(shape: dict, layers: int, dtype: str, max_requests: int, num_pages: int, graphs: bool):
    import torch

    from pylon_amd.config import resolve
    from pylon_amd.engine import Model, Runner, resolve_dtype
    from pylon_amd.weights import fill_random_model

    raw = config_json(shape, layers)
    arch = resolve(raw)
    cfg = arch.parse_config(raw)
    model = Model(arch.model_spec(cfg), dtype=resolve_dtype(dtype), device="cuda:0")
    fill_random_model(model, arch, cfg, seed=0, std=0.02)  # the random-weights mode, on the device
    runner = Runner(model, page_size=PAGE_SIZE, num_pages=num_pages, max_requests=max_requests)
    if graphs:
        runner.enable_graphs(max_requests, max_tokens_per_request=shape["max_position_embeddings"])
    torch.cuda.synchronize()
    return runner, cfg


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


def feed_prompts(runner, sampler, seqs, prompts) -> None:
    """The prompts through the step function in steps of at most PREFILL_TOKENS tokens, cut by
    the scheduler's own rule (:func:`pylon_amd.engine.scheduler.cut_prompts`: short prompts
    side by side, a long one in portions); the first new token of each request is chosen on
    the device."""
    from pylon_amd.engine import StepEntry
    from pylon_amd.engine.scheduler import PromptWork, cut_prompts
    from pylon_amd.sampling import Sampling

    fed = [0] * len(seqs)
    while True:
        work = [PromptWork(i, len(prompts[i]) - fed[i], 0.0) for i in range(len(seqs)) if fed[i] < len(prompts[i])]
        portions = cut_prompts(work, PREFILL_TOKENS, 0.0)
        if not portions:
            return
        entries = []
        for i, take in portions:
            last = fed[i] + take == len(prompts[i])
            entries.append(StepEntry(seqs[i], prompts[i][fed[i]: fed[i] + take], [take - 1] if last else []))
            fed[i] += take
        out = runner.step(entries)
        wanted = sum(len(e.want) for e in entries)
        if wanted:
            greedy = [(Sampling(temperature=0.0), 0)] * wanted
            sampler.launch(out, greedy, chosen=runner.chosen, place=runner.logit_slots).result()


def decode_run(runner, cfg, batch: int, steps: int, warmup: int, seed: int, prompt_len: int = PROMPT_LEN):
    """Prefill ``batch`` prompts of ``prompt_len`` random ids, then time ``steps`` decode steps."""
    import numpy as np
    import torch

    from pylon_amd.engine import PENDING, StepEntry
    from pylon_amd.sampling import Sampler, Sampling

    sampler = Sampler(runner.model.device)
    greedy = [(Sampling(temperature=0.0), 0)] * batch
    rng = np.random.default_rng(seed)
    seqs = [runner.open(f"b{batch}-{i}") for i in range(batch)]
    prompts = [rng.integers(0, cfg.vocab_size, prompt_len).tolist() for _ in range(batch)]
    feed_prompts(runner, sampler, seqs, prompts)

    entries = [StepEntry(seqs[i], [PENDING], [0]) for i in range(batch)]
    produced = []

    def one_step(before):
        out = runner.step(entries)
        draw = sampler.launch(out, greedy, chosen=runner.chosen, place=runner.logit_slots)
        if before is not None:
            produced.append(before.result())
        return draw

    draw = None
    for _ in range(warmup):
        draw = one_step(draw)
    torch.cuda.synchronize()
    context_sum = 0
    started = time.perf_counter()
    for _ in range(steps):
        context_sum += sum(s.length + 1 for s in seqs)
        draw = one_step(draw)
    produced.append(draw.result())
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    assert len(produced) == warmup + steps and all(len(p) == batch for p in produced)
    for s in seqs:
        runner.close(s)
    return elapsed, context_sum / steps  # seconds, mean cached tokens read per step (all rows)


def prefill_run(runner, cfg, repeats: int, seed: int):
    """One prompt of PREFILL_TOKENS random ids in one step; the median of ``repeats`` runs."""
    import numpy as np
    import torch

    from pylon_amd.engine import StepEntry

    rng = np.random.default_rng(seed)
    times = []
    for r in range(repeats + 1):
        seq = runner.open(f"prefill-{r}")
        prompt = rng.integers(0, cfg.vocab_size, PREFILL_TOKENS).tolist()
        torch.cuda.synchronize()
        started = time.perf_counter()
        out = runner.step([StepEntry(seq, prompt, [PREFILL_TOKENS - 1])])
        out.cpu()
        times.append(time.perf_counter() - started)
        runner.close(seq)
    times = sorted(times[1:])  # the first run warms the library's kernels up
    return times[len(times) // 2]


def mixed_run(runner, cfg, batch: int, prompt_len: int, repeats: int, seed: int) -> float:
    """Seconds of one mixed step: one token for each of ``batch`` requests that hold
    ``prompt_len`` tokens, beside a PREFILL_TOKENS portion of a new prompt, with greedy
    sampling of the batch + 1 wanted rows on the device; the median."""
    import numpy as np
    import torch

    from pylon_amd.engine import StepEntry
    from pylon_amd.sampling import Sampler, Sampling

    rng = np.random.default_rng(seed)
    sampler = Sampler(runner.model.device)
    greedy = [(Sampling(temperature=0.0), 0)] * (batch + 1)
    seqs = [runner.open(f"m{batch}-{i}") for i in range(batch)]
    feed_prompts(runner, sampler, seqs, [rng.integers(0, cfg.vocab_size, prompt_len).tolist() for _ in seqs])
    times = []
    for r in range(repeats + 1):
        fresh = runner.open(f"mixed-prompt-{r}")
        entries = [StepEntry(s, [int(rng.integers(0, cfg.vocab_size))], [0]) for s in seqs]
        entries.append(StepEntry(fresh, rng.integers(0, cfg.vocab_size, PREFILL_TOKENS).tolist(), [PREFILL_TOKENS - 1]))
        torch.cuda.synchronize()
        started = time.perf_counter()
        out = runner.step(entries)
        sampler.launch(out, greedy, chosen=runner.chosen, place=runner.logit_slots).result()
        times.append(time.perf_counter() - started)
        runner.close(fresh)
    for s in seqs:
        runner.close(s)
    times = sorted(times[1:])
    return times[len(times) // 2]


def engine_run(runner, cfg, batch: int, seed: int, prompt_len: int = PROMPT_LEN, new_tokens: int = NEW_TOKENS):
    """The same work through the scheduler: ``batch`` requests of ``prompt_len`` random ids and
    ``new_tokens`` greedy tokens each, queued at once; generated tokens per second from the
    first request's arrival to the last one's end (admission, the prompts' prefill, ticks,
    sampling and the host's reading of every token included), and the median time from a
    request's arrival to its first token in milliseconds."""
    import numpy as np
    import torch

    from pylon_amd.config import PylonConfig
    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    rng = np.random.default_rng(seed)
    prompts = [rng.integers(0, cfg.vocab_size, prompt_len).tolist() for _ in range(batch)]
    engine = Engine(PylonConfig(max_batch_size=batch, max_queue_size=batch, page_size=PAGE_SIZE), runner=runner)
    sampling = Sampling(max_new_tokens=new_tokens, temperature=0.0)
    if runner.graphs is not None:  # as a server does at start-up
        longest = prompt_len + new_tokens
        runner.capture_graphs(range(1, batch + 1),
                              bounds=[b for b in runner.graphs.bounds() if b < 2 * longest])
    torch.cuda.synchronize()
    started = time.perf_counter()
    results = engine.generate(prompts, sampling)
    elapsed = time.perf_counter() - started
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
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--no-graphs", action="store_true", help="launch decode steps kernel by kernel")
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
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

    shape = SHAPES[args.shape]
    layers = args.layers or shape["num_hidden_layers"]
    context_length = shape["max_position_embeddings"]
    prompt_len = args.prompt_len
    steps = min(args.steps, context_length - prompt_len - args.warmup)
    max_batch = args.batch if args.no_points else max(64, args.batch)
    # The pool holds a whole context for every request where that stays under a third of the
    # card's memory, else what the longest run here needs.
    element = 2 if args.dtype == "bfloat16" else 4
    page_bytes = 2 * layers * PAGE_SIZE * shape["num_key_value_heads"] * shape["head_dim"] * element
    pages_per_request = context_length // PAGE_SIZE
    if max_batch * pages_per_request * page_bytes > 100e9:
        longest = max(prompt_len + steps + args.warmup + 1, PREFILL_TOKENS)
        pages_per_request = -(-longest // PAGE_SIZE) + 1
    runner, cfg = build_runner(shape, layers, args.dtype, max_requests=max_batch + 1,
                               num_pages=(max_batch + 1) * pages_per_request, graphs=not args.no_graphs)
    dtype_key = "bf16" if args.dtype == "bfloat16" else "fp32"
    if args.prefill_only:
        seconds = prefill_run(runner, cfg, repeats=5, seed=2)
        print(json.dumps({"prefill": {"value": round(PREFILL_TOKENS / seconds, 1), "tokens": PREFILL_TOKENS,
                                      "ms": round(1e3 * seconds, 3)}}))
        return 0

    elapsed, mean_context = decode_run(runner, cfg, args.batch, steps, args.warmup, seed=1, prompt_len=prompt_len)
    ms_per_step = 1e3 * elapsed / steps
    value = args.batch * steps / elapsed
    per_token = runner.manager.bytes_per_token
    step_bytes = weight_bytes(runner) + mean_context * per_token
    achieved = step_bytes / (elapsed / steps)

    headline = (args.shape == "4b" and args.batch == 8 and prompt_len == PROMPT_LEN and args.dtype == "bfloat16"
                and layers == shape["num_hidden_layers"])
    record = {
        "metric": f"decode tokens/s, Qwen3-{args.shape.upper()} shape, batch {args.batch}, {prompt_len}-token prompts",
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
            "hip_graphs": runner.graphs is not None, "parallelism": "single-gpu",
            "baseline": "reference on one NVIDIA L4, 8 clients: 199.8 tokens/s",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_BYTES_PER_S / 1e9,
                     "unit": "GB/s", "frac": round(achieved / HBM_BYTES_PER_S, 4)},
    }
    if not args.no_prefill:
        seconds = prefill_run(runner, cfg, repeats=5, seed=2)
        attention = 4.0 * cfg.num_hidden_layers * cfg.num_attention_heads * cfg.head_dim * (
            PREFILL_TOKENS * (PREFILL_TOKENS + 1) / 2)
        flops = linear_flops_per_token(cfg) * PREFILL_TOKENS + attention + 2.0 * cfg.hidden_size * cfg.vocab_size
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
    if args.mixed:
        seconds = mixed_run(runner, cfg, args.batch, prompt_len, repeats=5, seed=4)
        record["mixed"] = {"decodes": args.batch, "chunk": PREFILL_TOKENS, "ms": round(1e3 * seconds, 3)}
    if not args.no_points:
        points = {}
        for batch in (1, 64):
            n = min(steps, 256)
            e, _ = decode_run(runner, cfg, batch, n, args.warmup, seed=3 + batch, prompt_len=prompt_len)
            points[f"decode_b{batch}"] = round(batch * n / e, 1)
        rate, first_ms = engine_run(runner, cfg, batch=8, seed=9, prompt_len=prompt_len)
        points["engine_b8"], points["engine_b8_first_token_ms"] = round(rate, 1), round(first_ms, 2)
        # the reference's other published workload: 2,048-token prompts, 32 new tokens, 8 at a time
        # (53.7 output tokens/s and 847 ms to the first token on its L4, /root/reference/README.md:76,90)
        rate, first_ms = engine_run(runner, cfg, batch=8, seed=10, prompt_len=PREFILL_TOKENS, new_tokens=32)
        points["engine_prefill_heavy_b8"] = round(rate, 1)
        points["engine_prefill_heavy_b8_first_token_ms"] = round(first_ms, 2)
        record["points"] = points
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
