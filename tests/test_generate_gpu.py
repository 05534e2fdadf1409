"""Generation through the entry point against the plain implementation: greedy, seeded
temperature sampling, the first tokens of a sequence, and long decoding."""
import numpy as np
import pytest
import torch

from tests.helpers import make_model_folder, random_tokens, read_folder
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tmp(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return tmp_path_factory.mktemp("gen")


def plain_generate(weights, cfg, prompt, count, pick):
    tokens = list(prompt)
    out = []
    for i in range(count):
        nxt = pick(plain.forward(weights, cfg, tokens)[-1], i)
        out.append(nxt)
        tokens.append(nxt)
    return out


def margins_ok(weights, cfg, prompt, produced, floor):
    """True if every greedy choice of the plain model wins by more than ``floor``."""
    tokens = list(prompt)
    for tok in produced:
        row = np.sort(plain.forward(weights, cfg, tokens)[-1])
        if row[-1] - row[-2] <= floor:
            return False
        tokens.append(tok)
    return True


def follows_plain(weights, cfg, prompt, produced, slack):
    """Every produced token is the plain model's greedy choice given the tokens before it (the
    produced ones, so that one flipped near-tie does not excuse what follows), or loses to
    that choice by no more than ``slack`` times the row's largest |logit|.  Returns the index
    of the first token that is neither, or None."""
    tokens = list(prompt)
    for i, tok in enumerate(produced):
        row = plain.forward(weights, cfg, tokens)[-1]
        if tok != int(row.argmax()) and row.max() - row[tok] > slack * np.abs(row).max():
            return i
        tokens.append(tok)
    return None


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(tmp, dtype):
    """Tiny A's workload: prompts of 5, 17 and 33 tokens, 16 greedy tokens each, all three
    running together through the scheduler with prompts cut into portions of 8."""
    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    folder = make_model_folder(tmp, "A", dtype=dtype, std=0.08)
    cfg, weights = read_folder(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, 70 + n) for n in (5, 17, 33)]
    engine = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=12, max_batch_size=4,
                                prefill_chunk_size=8)
    try:
        results = engine.generate(prompts, Sampling(max_new_tokens=16, temperature=0.0))
    finally:
        engine.close()
    assert engine.runner.manager.free_pages == 12
    for prompt, result in zip(prompts, results):
        want = plain_generate(weights, cfg, prompt, 16, lambda row, i: plain.greedy(row))
        assert result.finish_reason == "length" and len(result.output_ids) == 16
        if dtype == "float32":
            assert result.output_ids == want
        else:
            # bfloat16 may flip a near-tie: every token, given the engine's own tokens before
            # it, must be the plain model's choice or within the logits' error bound of it
            assert follows_plain(weights, cfg, prompt, result.output_ids, 2e-2) is None
            agree = next((i for i, (a, b) in enumerate(zip(result.output_ids, want)) if a != b), 16)
            assert agree == 16 or not margins_ok(weights, cfg, prompt, want[: agree + 1], 0.02)


def test_the_threaded_engine_on_the_gpu(tmp):
    """The background thread drives the real step function while requests arrive from this
    thread; results are the plain model's greedy tokens (float32: exactly)."""
    import time

    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    folder = make_model_folder(tmp, "B", dtype="float32", std=0.08)
    cfg, weights = read_folder(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, 300 + n) for n in (3, 40, 9, 21, 2, 65)]
    engine = Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=40, max_batch_size=3,
                                prefill_chunk_size=16, threaded=True)
    try:
        futures = []
        for prompt in prompts:
            futures.append(engine.enqueue(prompt, None, Sampling(max_new_tokens=6, temperature=0.0)))
            time.sleep(0.002)  # arrivals spread over the ticks
            assert set(engine.snapshot()) >= {"waiting", "active"}
        results = [f.result(timeout=60) for f in futures]
    finally:
        engine.close()
    for prompt, result in zip(prompts, results):
        assert result.output_ids == plain_generate(weights, cfg, prompt, 6, lambda row, i: plain.greedy(row))
        assert result.first_token_seconds is not None and len(result.token_intervals) == 5
    assert engine.runner.manager.free_pages == 40


def test_stop_token_and_first_token_from_a_one_token_prompt(tmp):
    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    folder = make_model_folder(tmp, "B", dtype="float32", std=0.08)
    cfg, weights = read_folder(folder)
    prompt = [7]
    want = plain_generate(weights, cfg, prompt, 8, lambda row, i: plain.greedy(row))
    engine = Engine.from_folder(folder, dtype="float32", page_size=32, num_pages=4)
    try:
        got = engine.generate([prompt], Sampling(max_new_tokens=8, temperature=0.0))[0]
        assert got.output_ids == want
        stop = want[3]
        first = want.index(stop)
        cut = engine.generate([prompt], Sampling(max_new_tokens=8, temperature=0.0), eos_token_id=stop)[0]
        assert cut.finish_reason == "eos" and cut.output_ids == want[:first]
    finally:
        engine.close()


def test_seeded_temperature_sampling_matches_the_plain_rule(tmp):
    """Tiny B's workload: prompts of 1, 31, 64 and 100 tokens in portions of 48 beside
    decodes, temperature 0.8 from a fixed seed, 24 tokens each.  The engine's draw for
    token i of a request is the cumulative distribution read at uniform(seed, i)."""
    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling, uniform

    folder = make_model_folder(tmp, "B", dtype="float32", std=0.08)
    cfg, weights = read_folder(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, 90 + n) for n in (1, 31, 64, 100)]
    for top_p in (1.0, 0.9):
        sampling = Sampling(max_new_tokens=24, temperature=0.8, top_p=top_p, seed=1234)
        engine = Engine.from_folder(folder, dtype="float32", page_size=32, num_pages=16,
                                    max_batch_size=4, prefill_chunk_size=48)
        try:
            results = engine.generate(prompts, sampling)
            alone = engine.generate([prompts[2]], sampling)[0]
        finally:
            engine.close()
        # a request's tokens do not depend on what ran beside it
        assert alone.output_ids == results[2].output_ids
        for prompt, result in zip(prompts, results):
            tokens = list(prompt)
            for i, tok in enumerate(result.output_ids):
                row = plain.forward(weights, cfg, tokens)[-1]
                u = uniform(1234, i)
                want = plain.sample_with_uniform(row, 0.8, top_p, u)
                if tok != want:
                    p = plain.sampling_distribution(row, 0.8, top_p)
                    cdf = np.cumsum(p)
                    assert p[tok] > 0 and abs(cdf[min(tok, want)] - u) < 1e-4, (i, tok, want)
                tokens.append(tok)
        assert len({tuple(r.output_ids) for r in results}) == 4


def test_long_decoding_stays_on_the_plain_model(tmp):
    """600 tokens decoded one by one after a short prompt (crossing many pages), with the
    logits of the engine's own token sequence compared at the end."""
    from pylon_amd.engine import Runner, StepEntry

    folder = make_model_folder(tmp, "C", dtype="float32", std=0.08)
    cfg, weights = read_folder(folder)
    prompt = random_tokens(cfg["vocab_size"], 11, 3)
    runner = Runner.from_folder(folder, dtype="float32", page_size=64, num_pages=10, max_requests=2)
    seq = runner.open("long")
    logits = runner.step([StepEntry(seq, prompt, [len(prompt) - 1])])
    tokens, rows = list(prompt), []
    for _ in range(600):
        rows.append(logits[0].cpu().numpy())
        nxt = int(torch.argmax(logits[0]).item())
        tokens.append(nxt)
        logits = runner.step([StepEntry(seq, [nxt], [0])])
    assert seq.length == 611 and len(seq.pages[0]) == 10
    want = plain.forward(weights, cfg, tokens[:-1])[len(prompt) - 1:]
    got = np.stack(rows)
    err = np.abs(got - want).max(axis=1)
    assert err.max() <= 2e-5 * np.abs(want).max(), int(err.argmax())
    assert len(set(tokens[len(prompt):])) > 3  # the model does not just repeat one token


@pytest.mark.parametrize("graphs", [False, True])
def test_running_ahead_gives_the_tokens_of_the_tick_by_tick_engine(tmp, graphs):
    """The same requests (greedy and seeded sampling, with a stop token) with and without
    the next step queued before the last one's tokens are read."""
    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    folder = make_model_folder(tmp, "A", dtype="bfloat16", std=0.08)
    cfg, _ = read_folder(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, 30 + n) for n in (3, 9, 20, 41)]
    outputs = []
    for ahead in (False, True):
        engine = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=24, max_batch_size=4,
                                    prefill_chunk_size=16, run_ahead=ahead, cuda_graphs=graphs)
        assert engine._run_ahead == ahead
        try:
            greedy = engine.generate(prompts, Sampling(max_new_tokens=40, temperature=0.0))
            stop = greedy[1].output_ids[7]
            cut = engine.generate(prompts, Sampling(max_new_tokens=40, temperature=0.0), eos_token_id=stop)
            drawn = engine.generate(prompts, Sampling(max_new_tokens=40, temperature=0.9, top_p=0.9, seed=5))
        finally:
            engine.close()
        assert engine.runner.manager.free_pages == 24
        engine.runner.manager.check()
        if graphs:
            assert engine.runner.graphs.replays > 0
        outputs.append([(r.output_ids, r.finish_reason) for r in greedy + cut + drawn])
        assert any(reason == "eos" for _, reason in outputs[-1])
    assert outputs[0] == outputs[1]


def test_random_weights_straight_into_an_engine_and_the_command_line(tmp, tmp_path):
    """Engine.from_random(config, seed, draw_on="cpu") is the engine over the folder that the
    random-weights mode writes from the same (config, seed); drawn on the GPU (the default) the
    numbers are others, the same on every run; `main.py generate --random` prints its tokens."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling
    from tests.helpers import CONFIGS, NORM_JITTER, SEEDS

    folder = make_model_folder(tmp, "D", dtype="bfloat16")
    prompt = random_tokens(CONFIGS["D"]["vocab_size"], 12, 3)
    sampling = Sampling(max_new_tokens=10, temperature=0.0)
    outputs = []
    for make in (lambda: Engine.from_folder(folder, dtype="bfloat16", page_size=64, num_pages=4),
                 lambda: Engine.from_random(CONFIGS["D"], SEEDS["D"], norm_jitter=NORM_JITTER["D"], draw_on="cpu",
                                            dtype="bfloat16", page_size=64, num_pages=4)):
        engine = make()
        try:
            outputs.append(engine.generate([prompt], sampling)[0].output_ids)
        finally:
            engine.close()
    assert outputs[0] == outputs[1] and len(outputs[0]) == 10
    config_file = tmp_path / "config.json"
    config_file.write_text(json.dumps(CONFIGS["D"]))
    root = Path(__file__).resolve().parent.parent
    done = subprocess.run(
        [sys.executable, str(root / "main.py"), "generate", "--random", str(config_file), "--seed", str(SEEDS["D"]),
         "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "10", "--temperature", "0",
         "--page-size", "64", "--num-pages", "4"],
        capture_output=True, text=True, timeout=120, cwd=str(tmp_path))
    assert done.returncode == 0, done.stderr[-2000:]
    line = json.loads(done.stdout.strip().splitlines()[-1])
    # the command line draws unit norm weights (no jitter): the same as from_random without it
    engine = Engine.from_random(CONFIGS["D"], SEEDS["D"], dtype="bfloat16", page_size=64, num_pages=4)
    try:
        want = engine.generate([prompt], sampling)[0].output_ids
    finally:
        engine.close()
    assert line["output_ids"] == want and line["finish_reason"] == "length"


def test_a_random_workload_gives_the_same_tokens_in_every_mode_of_the_engine(tmp):
    """Fifty requests of random lengths, greedy and seeded sampling, half of them with a stop
    token that they really meet, through the scheduler with few pages and slots: tick by
    tick or running ahead, kernel by kernel or from graphs, every request's tokens are the
    same (float32 kernels do not depend on what shares a batch)."""
    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    folder = make_model_folder(tmp, "D", dtype="float32", std=0.08)
    cfg, _ = read_folder(folder)
    rng = np.random.default_rng(5)
    requests = []
    for i in range(50):
        prompt = rng.integers(0, cfg["vocab_size"], int(rng.integers(1, 260))).tolist()
        sampling = Sampling(max_new_tokens=int(rng.integers(1, 40)), temperature=float(rng.choice([0.0, 0.8])),
                            top_p=0.9, seed=i)
        requests.append((prompt, sampling))

    def run(stops, **options):
        engine = Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=60, max_batch_size=6,
                                    prefill_chunk_size=64, max_queue_size=64, **options)
        try:
            futures = [engine.enqueue(p, stop, s, f"r{i}") for i, ((p, s), stop) in enumerate(zip(requests, stops))]
            engine.run_until_idle()
            results = [f.result(timeout=0) for f in futures]
        finally:
            engine.close()
        assert engine.runner.manager.free_pages == 60
        engine.runner.manager.check()
        return [(r.output_ids, r.finish_reason) for r in results]

    free = run([None] * len(requests))
    stops = [out[4] if i % 2 == 0 and len(out) > 4 else None for i, (out, _) in enumerate(free)]
    base = run(stops, run_ahead=False)
    assert sum(reason == "eos" for _, reason in base) >= 10
    for options in (dict(run_ahead=True), dict(run_ahead=False, cuda_graphs=True), dict(run_ahead=True, cuda_graphs=True)):
        assert run(stops, **options) == base, options
