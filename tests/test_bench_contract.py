"""What `bench.py` promises whoever drives it, as far as a machine without a GPU can tell: one
GPU only (any other count: one line and exit status 2), the layer sizes of the benchmark
configuration, and the counts of bytes and operations its fractions are made from."""
import importlib.util
import json
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", ROOT / "bench.py")
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def test_more_than_one_gpu_is_one_line_and_status_2():
    for count in ("2", "8", "0"):
        run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", count, "--steps", "3", "--warmup", "1"],
                             capture_output=True, text=True, timeout=120)
        assert run.returncode == 2, (count, run.returncode, run.stderr[-300:])
        assert len(run.stdout.strip().splitlines()) == 1 and "one GPU" in run.stdout


def test_the_default_shape_is_the_benchmark_configuration():
    bench = _bench()
    shape = bench.SHAPES["4b"]
    assert (shape["num_hidden_layers"], shape["hidden_size"], shape["num_attention_heads"],
            shape["num_key_value_heads"], shape["head_dim"], shape["intermediate_size"], shape["vocab_size"],
            shape["max_position_embeddings"]) == (36, 2560, 32, 8, 128, 9728, 151936, 8192)
    assert shape["rope_theta"] == 5e6 and shape["tie_word_embeddings"] is True
    named = json.loads((ROOT / "BASELINE.json").read_text())["configs"][2]
    for size in ("36 layers", "hidden 2560", "32 heads", "8 KV heads", "head_dim 128", "intermediate 9728",
                 "vocab 151936", "Context length 8192", "256-token KV pages"):
        assert size in named, size
    assert bench.PAGE_SIZE == 256 and bench.PREFILL_TOKENS == 2048 and bench.PROMPT_LEN == 128
    # the published peaks the fractions are taken against
    assert bench.HBM_BYTES_PER_S == 8e12
    raw = bench.config_json(shape, 36)
    assert raw["architectures"] == ["Qwen3ForCausalLM"] and raw["num_hidden_layers"] == 36


def test_operation_counts():
    """Two operations per weight of the layers per token (the head is taken at a prompt's last
    row only and not counted); attention: for every new token the keys before it and itself,
    scores and values, every head."""
    bench = _bench()

    class Cfg:
        num_hidden_layers, hidden_size, num_attention_heads, num_key_value_heads = 36, 2560, 32, 8
        head_dim, intermediate_size, vocab_size = 128, 9728, 151936

    per_layer = 2560 * (32 + 16) * 128 + 32 * 128 * 2560 + 3 * 2560 * 9728
    assert bench.linear_flops_per_token(Cfg) == 2.0 * 36 * per_layer
    whole = bench.attention_flops(Cfg, 2048)
    assert whole == 36 * 32 * 128 * 4.0 * (2048 * 2049 / 2)
    assert bench.attention_flops(Cfg, 1, cached=4095) == 36 * 32 * 128 * 4.0 * 4096
