"""Start-up as a server does it: the page pool sized from the device's memory (no
``num_pages``), the refusal of weights that do not fit, and decode graphs captured at
start-up for a model whose position limit is 262,144 tokens
(/root/reference/src/pylon/kv/budget.py:49-113, /root/reference/src/pylon/decode/warmup.py:140-167)."""
import time

import numpy as np
import pytest
import torch

from tests.helpers import CONFIGS, make_model_folder, random_tokens, read_folder
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")


def test_the_pool_is_sized_from_device_memory(gpu, tmp_path):
    from pylon_amd.config import PylonConfig
    from pylon_amd.engine.engine import Engine
    from pylon_amd.engine.runner import pool_pages
    from pylon_amd.sampling import Sampling

    folder = make_model_folder(tmp_path, "D", dtype="bfloat16", std=0.08)
    cfg, weights = read_folder(folder)
    free, total = torch.cuda.mem_get_info()
    # (a) plenty of memory: the pool is what max_batch_size requests of the longest length hold
    engine = Engine.from_folder(folder, max_batch_size=3, page_size=64)
    try:
        sizing = engine.runner.pool_sizing
        assert sizing is not None and sizing["bytes_per_token"] == 2 * 2 * 2 * 64 * 2
        assert engine.runner.manager.num_pages == sizing["num_pages"] == 3 * (4096 // 64)
        prompt = random_tokens(cfg["vocab_size"], 33, 5)
        result, = engine.generate([prompt], Sampling(max_new_tokens=6, temperature=0.0))
        ref = list(prompt)
        for got in result.output_ids:
            row = plain.forward(weights, cfg, ref)[-1]
            best = np.sort(row)
            assert got == int(row.argmax()) or best[-1] - row[got] <= 2e-2 * np.abs(row).max()
            ref.append(got)
    finally:
        engine.close()
    # (b) memory is the limit: a utilisation limit that leaves a few megabytes
    occupied = total - torch.cuda.mem_get_info()[0]
    tight = (occupied + (64 << 20)) / total
    engine = Engine.from_folder(folder, max_batch_size=32, page_size=64, max_gpu_utilization=tight,
                                weight_headroom_ratio=0.0, kv_cache_headroom_ratio=0.0, cuda_graphs=True)
    try:
        sizing = engine.runner.pool_sizing
        config = PylonConfig(max_batch_size=32, page_size=64, max_gpu_utilization=tight,
                             kv_cache_headroom_ratio=0.0)
        # the headroom is the measured peak of the largest step these options allow, not a ratio
        assert 0 < sizing["activation_bytes"] < 64 << 20
        expected = pool_pages(sizing["free"], sizing["total"], sizing["bytes_per_token"], config, 4096,
                              activation_bytes=sizing["activation_bytes"])
        assert engine.runner.manager.num_pages == sizing["num_pages"] == expected
        assert 1 <= expected < 32 * (4096 // 64)  # below the ceiling: memory decided
        pool_bytes = expected * 64 * sizing["bytes_per_token"]
        assert pool_bytes <= 64 << 20
        results = engine.generate([random_tokens(cfg["vocab_size"], n, n) for n in (9, 40)],
                                  Sampling(max_new_tokens=5, temperature=0.0))
        assert all(len(r.output_ids) == 5 for r in results)
        assert engine.runner.graphs.replays > 0
    finally:
        engine.close()
    # (c) weights that do not fit under the limit are refused before anything is loaded
    with pytest.raises(RuntimeError, match="Refusing to load"):
        Engine.from_folder(folder, max_gpu_utilization=1e-9)


LONG = dict(CONFIGS["D"], max_position_embeddings=262144, num_hidden_layers=3, vocab_size=1531)


def test_start_up_with_graphs_at_a_position_limit_of_262144(gpu, tmp_path):
    """Every decode graph is captured at start-up, in bounded time and memory: bounds on the
    requests' lengths at which the recorded launches are the same share a graph, so ten bounds
    make a few graphs per small batch size and two per large one; no graph is captured while
    serving, however long the request."""
    from pylon_amd.engine.engine import Engine
    from pylon_amd.engine import StepEntry
    from pylon_amd.kernels import ops

    folder = make_model_folder(tmp_path, "long", dtype="bfloat16", config=LONG, std=0.08)
    cfg, weights = read_folder(folder)
    torch.cuda.synchronize()
    before = torch.cuda.memory_reserved()
    started = time.perf_counter()
    engine = Engine.from_folder(folder, cuda_graphs=True, max_batch_size=32)
    elapsed = time.perf_counter() - started
    try:
        runner = engine.runner
        graphs = runner.graphs
        assert len(graphs.bounds()) == 10 and graphs.bounds()[0] == 512 and graphs.bounds()[-1] == 262144
        expected = {(rows, (("attention", *ops.decode_launch(rows, cfg["num_key_value_heads"], bound)),))
                    for rows in range(1, 33) for bound in graphs.bounds()}
        assert set(graphs.captured) == expected
        assert 32 < len(expected) < 32 * 4  # far fewer than one per batch size and bound (320)
        assert runner.manager.num_pages == 32 * (262144 // 256)
        pool = runner.manager.num_pages * 256 * runner.manager.bytes_per_token
        extra = torch.cuda.memory_reserved() - before - pool
        print(f"start-up {elapsed:.1f} s ({runner.startup}); {len(expected)} graphs and their buffers hold "
              f"{extra / 2**20:.0f} MiB")
        assert elapsed < 90 and extra < 768 << 20
        # a request longer than 1,024 tokens replays a graph that is already there
        prompt = random_tokens(cfg["vocab_size"], 1030, 9)
        seq = runner.open("long")
        runner.step([StepEntry(seq, prompt, [])])
        tail = random_tokens(cfg["vocab_size"], 3, 10)
        replays = graphs.replays
        rows = [runner.step([StepEntry(seq, [t], [0])]).cpu().numpy()[0] for t in tail]
        runner.close(seq)
        assert set(graphs.captured) == expected and graphs.replays == replays + 3
        want = plain.forward(weights, cfg, prompt + tail)[-3:]
        for got, ref in zip(rows, want):
            assert np.abs(got - ref).max() <= 2e-2 * np.abs(ref).max()
    finally:
        engine.close()


def test_start_up_captures_graphs_up_to_a_configured_length(gpu, tmp_path):
    """``cuda_graph_max_tokens`` bounds what start-up captures; a longer request's graph is
    captured when it first decodes."""
    from pylon_amd.engine.engine import Engine
    from pylon_amd.engine import StepEntry

    folder = make_model_folder(tmp_path, "long", dtype="bfloat16", config=LONG, std=0.08)
    cfg, _ = read_folder(folder)
    engine = Engine.from_folder(folder, cuda_graphs=True, max_batch_size=4, cuda_graph_max_tokens=1000,
                                num_pages=64)
    try:
        graphs = engine.runner.graphs
        assert set(graphs.captured) == {graphs.key(rows, bound) for rows in range(1, 5) for bound in (512, 1024)}
        seq = engine.runner.open("long")
        engine.runner.step([StepEntry(seq, random_tokens(cfg["vocab_size"], 2100, 9), [])])
        engine.runner.step([StepEntry(seq, [5], [0])])
        engine.runner.close(seq)
        assert graphs.key(1, 4096) in graphs.captured and len(graphs.captured) == 9
    finally:
        engine.close()


def test_a_bfloat16_model_over_a_folder_stored_in_32_bit(gpu, tmp_path, caplog):
    """Matrices stored in 32-bit stay 32-bit in a bfloat16 model: start-up counts them at four
    bytes an element, says so, and the steps (bfloat16 activations times float32 matrices, on
    the exact product kernel) match the plain model."""
    from pylon_amd.engine.engine import Engine
    from pylon_amd.engine import StepEntry
    from pylon_amd.engine.runner import weight_bytes

    folder = make_model_folder(tmp_path, "D", dtype="float32", std=0.08)
    cfg, weights = read_folder(folder)
    with caplog.at_level("WARNING", logger="pylon"):
        engine = Engine.from_folder(folder, dtype="bfloat16", page_size=64, max_batch_size=2, cuda_graphs=True)
    try:
        assert "weights_kept_32bit" in caplog.text
        model = engine.runner.model
        assert model.params["embed"].dtype == torch.float32 and model.dtype == torch.bfloat16
        assert engine.runner.manager.groups[0].k[0].dtype == torch.bfloat16
        real = sum(o.params[n].numel() * o.params[n].element_size() for _, o, n in model.named_params())
        assert real > 1.9 * weight_bytes(model.spec, torch.bfloat16)
        prompt = random_tokens(cfg["vocab_size"], 150, 4)
        want = plain.forward(weights, cfg, prompt + [7, 8])
        seq = engine.runner.open("r")
        replays = engine.runner.graphs.replays  # start-up's captures count as replays
        got = [engine.runner.step([StepEntry(seq, prompt, list(range(150)))]).cpu().numpy()]
        got += [engine.runner.step([StepEntry(seq, [t], [0])]).cpu().numpy() for t in (7, 8)]
        engine.runner.close(seq)
        assert engine.runner.graphs.replays == replays + 2
        got = np.concatenate(got)
        frac = np.abs(got - want).max(axis=1) / np.abs(want).max(axis=1)
        assert frac.max() <= 2e-2, (int(frac.argmax()), float(frac.max()))
    finally:
        engine.close()


def test_random_weights_start_up_like_a_folder(gpu):
    """``Engine.from_random`` goes through the same start-up as a folder (fit check, measured
    headroom, sized pool, graphs) without writing one, and draws the same numbers every time."""
    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    prompt = random_tokens(CONFIGS["D"]["vocab_size"], 30, 1)
    outputs = []
    for _ in range(2):
        engine = Engine.from_random(CONFIGS["D"], 5, std=0.08, page_size=64, max_batch_size=3, cuda_graphs=True)
        try:
            runner = engine.runner
            assert runner.pool_sizing["num_pages"] == runner.manager.num_pages == 3 * (4096 // 64)
            assert runner.pool_sizing["activation_bytes"] > 0 and runner.startup["total_s"] > 0
            assert runner.graphs.captured_sizes() == (1, 2, 3)
            outputs.append(engine.generate([prompt], Sampling(max_new_tokens=6, temperature=0.0))[0].output_ids)
        finally:
            engine.close()
    assert outputs[0] == outputs[1] and len(outputs[0]) == 6
    with pytest.raises(RuntimeError, match="Refusing to load a model of random weights"):
        Engine.from_random(CONFIGS["D"], 5, max_gpu_utilization=1e-9)


def test_groups_of_runs_get_pages_of_their_own_at_start_up(gpu, tmp_path):
    """A toy architecture (Qwen3's parts, the first layer with a window of 40 tokens): the sized
    pool gives the windowed group only the pages it can ever use, the engine runs long
    requests side by side through it without running out, and the tokens are the plain model's."""
    import dataclasses

    from pylon_amd.config import register_architecture, unregister_architecture
    from pylon_amd.config.registry import Architecture
    from pylon_amd.engine.engine import Engine
    from pylon_amd.models import qwen3
    from pylon_amd.sampling import Sampling
    from pylon_amd.weights import write_random_model

    def model_spec(cfg):
        spec = qwen3.model_spec(cfg)
        layers = list(spec.layers)
        layers[0] = dataclasses.replace(layers[0], mixer=dataclasses.replace(layers[0].mixer, window=40))
        return dataclasses.replace(spec, layers=tuple(layers))

    arch = Architecture("ToyWindowedForCausalLM", qwen3.parse_config, model_spec, qwen3.weight_targets,
                        lambda cfg: dict(qwen3.config_to_json(cfg), architectures=["ToyWindowedForCausalLM"]))
    register_architecture(arch)
    try:
        config = dict(CONFIGS["C"], architectures=["ToyWindowedForCausalLM"])
        folder = write_random_model(tmp_path / "windowed", config, 9, dtype="float32", std=0.08, norm_jitter=0.2)
        cfg, weights = read_folder(folder)
        engine = Engine.from_folder(folder, dtype="float32", page_size=16, max_batch_size=3, prefill_chunk_size=32)
        try:
            manager = engine.runner.manager
            # the full group: three requests of 2,048 positions; the windowed one: per request the
            # pages of 40 + 32 tokens and one more
            assert engine.runner.pool_sizing["pages_per_group"] == [18, 3 * 128]
            assert [g.requirement.window for g in manager.groups] == [40, None]
            assert [g.pool.num_pages for g in manager.groups] == [18, 384] and manager.num_pages == 384
            prompts = [random_tokens(cfg["vocab_size"], n, 20 + n) for n in (210, 77, 300, 150)]
            results = engine.generate(prompts, Sampling(max_new_tokens=30, temperature=0.0))
            assert manager.groups[0].pool.free_pages == 18 and manager.groups[1].pool.free_pages == 384
            manager.check()
        finally:
            engine.close()
        for prompt, result in zip(prompts, results):
            assert len(result.output_ids) == 30
            ref = list(prompt)
            for got in result.output_ids:
                row = plain.forward(weights, cfg, ref, windows={0: 40})[-1]
                best = np.sort(row)
                assert got == int(row.argmax()) or best[-1] - row[got] <= 1e-4 * np.abs(row).max()
                ref.append(got)
    finally:
        unregister_architecture("ToyWindowedForCausalLM")
