"""Configuration parsing and the architecture registry."""
import dataclasses
import json

import pytest

from pylon_amd.config import (PylonConfig, get_config, load_model_config, register_architecture,
                              registered_architectures, resolve, unregister_architecture)
from pylon_amd.config.specs import ModelSpec, ScheduleEntry
from pylon_amd.models import qwen3
from tests.helpers import TINY_A, TINY_B

# The content of /root/reference/tests/fixtures/config.json (the Qwen3-4B-Instruct-2507
# config.json), which the reference's loader test parses
# (/root/reference/tests/test_loader.py:79-83).
REFERENCE_FIXTURE = {
    "architectures": ["Qwen3ForCausalLM"], "attention_bias": False, "attention_dropout": 0.0,
    "bos_token_id": 151643, "eos_token_id": 151645, "head_dim": 128, "hidden_act": "silu",
    "hidden_size": 2560, "initializer_range": 0.02, "intermediate_size": 9728,
    "max_position_embeddings": 262144, "max_window_layers": 36, "model_type": "qwen3",
    "num_attention_heads": 32, "num_hidden_layers": 36, "num_key_value_heads": 8,
    "rms_norm_eps": 1e-06, "rope_scaling": None, "rope_theta": 5000000, "sliding_window": None,
    "tie_word_embeddings": True, "torch_dtype": "bfloat16", "transformers_version": "4.51.0",
    "use_cache": True, "use_sliding_window": False, "vocab_size": 151936,
}


def test_reference_fixture_parses_to_its_values():
    cfg = resolve(REFERENCE_FIXTURE).parse_config(REFERENCE_FIXTURE)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads,
            cfg.head_dim, cfg.intermediate_size, cfg.vocab_size) == (36, 2560, 32, 8, 128, 9728, 151936)
    assert cfg.rope_theta == 5_000_000.0 and cfg.rms_norm_eps == 1e-6
    assert cfg.max_position_embeddings == 262_144 and cfg.tie_word_embeddings is True
    assert cfg.eos_token_id == (151645,)


@pytest.mark.parametrize("raw", [TINY_A, TINY_B])
def test_model_spec_takes_every_size_from_the_config(raw):
    arch = resolve(raw)
    cfg = arch.parse_config(raw)
    spec = arch.model_spec(cfg)
    assert isinstance(spec, ModelSpec)
    assert len(spec.layers) == raw["num_hidden_layers"] == len(spec.schedule)
    layer = spec.layers[-1]
    assert layer.mixer.n_heads == raw["num_attention_heads"]
    assert layer.mixer.n_kv_heads == raw["num_key_value_heads"]
    assert layer.mixer.head_dim == raw["head_dim"]
    assert layer.mixer.q_size == raw["num_attention_heads"] * raw["head_dim"]
    assert abs(layer.mixer.scale - raw["head_dim"] ** -0.5) < 1e-15
    assert layer.mixer.position.theta == raw["rope_theta"]
    assert layer.mixer.position.rotary_dim == raw["head_dim"]
    assert layer.mixer.qk_norm and layer.mixer.qk_norm_eps == raw["rms_norm_eps"]
    assert layer.mixer.window is None
    assert layer.feed_forward.intermediate_size == raw["intermediate_size"]
    assert layer.mixer_norm.eps == raw["rms_norm_eps"] == spec.final_norm.eps
    assert spec.vocab_size == raw["vocab_size"] and spec.tie_word_embeddings == raw["tie_word_embeddings"]
    assert spec.max_positions == raw["max_position_embeddings"]
    assert spec.resolved_schedule() == tuple((i, i, True) for i in range(raw["num_hidden_layers"]))
    # the config survives a round trip through config.json
    assert arch.parse_config(arch.config_to_json(cfg)) == cfg


@pytest.mark.parametrize("field,value", [
    ("model_type", "llama"), ("hidden_act", "gelu"), ("attention_bias", True),
    ("rope_scaling", {"type": "yarn"}), ("use_sliding_window", True), ("sliding_window", 4096),
    ("tie_word_embeddings", "yes"),
])
def test_unsupported_fields_are_rejected_by_name(field, value):
    raw = dict(REFERENCE_FIXTURE)
    raw[field] = value
    with pytest.raises(ValueError, match=f"Checkpoint config field {field} is not supported"):
        qwen3.parse_config(raw)


def test_missing_keys_and_bad_sizes():
    raw = dict(TINY_A)
    del raw["head_dim"], raw["rope_theta"]
    with pytest.raises(ValueError, match="head_dim, rope_theta"):
        qwen3.parse_config(raw)
    with pytest.raises(ValueError, match="divisible"):
        qwen3.parse_config(dict(TINY_A, num_key_value_heads=3))
    with pytest.raises(ValueError, match="even head dimension"):
        qwen3.parse_config(dict(TINY_A, head_dim=15))
    with pytest.raises(ValueError, match="positive integer"):
        qwen3.parse_config(dict(TINY_A, vocab_size=0))


def test_registry_unknown_and_custom_architecture(tmp_path):
    with pytest.raises(ValueError, match="Unknown architecture 'NopeForCausalLM'"):
        resolve({"architectures": ["NopeForCausalLM"]})
    with pytest.raises(ValueError, match="exactly one architecture"):
        resolve({"architectures": []})
    assert "Qwen3ForCausalLM" in registered_architectures()
    toy = dataclasses.replace(qwen3.QWEN3, name="ToyForCausalLM")
    register_architecture(toy)
    try:
        with pytest.raises(ValueError, match="already registered"):
            register_architecture(toy)
        (tmp_path / "config.json").write_text(json.dumps(dict(TINY_A, architectures=["ToyForCausalLM"])))
        arch, cfg = load_model_config(tmp_path)
        assert arch.name == "ToyForCausalLM" and cfg.hidden_size == 64
    finally:
        unregister_architecture("ToyForCausalLM")


def test_schedule_is_checked():
    arch = resolve(TINY_A)
    spec = arch.model_spec(arch.parse_config(TINY_A))
    twice = dataclasses.replace(spec, schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1, cache=1)))
    assert twice.resolved_schedule() == ((0, 0, True), (1, 1, True), (0, 2, True), (1, 1, False))
    with pytest.raises(ValueError, match="names layer 5"):
        dataclasses.replace(spec, schedule=(ScheduleEntry(5),)).resolved_schedule()
    with pytest.raises(ValueError, match="earlier run"):
        dataclasses.replace(spec, schedule=(ScheduleEntry(0, cache=1), ScheduleEntry(1))).resolved_schedule()
    with pytest.raises(ValueError, match="borrows another"):
        dataclasses.replace(spec, schedule=(ScheduleEntry(0), ScheduleEntry(1, cache=0), ScheduleEntry(0, cache=1))).resolved_schedule()


def test_serving_config_defaults_and_checks(monkeypatch):
    cfg = PylonConfig()
    # the reference's defaults (/root/reference/src/pylon/config.py:14-26)
    assert (cfg.prefill_chunk_size, cfg.max_batch_size, cfg.max_queue_size, cfg.batch_wait_ms,
            cfg.max_gpu_utilization, cfg.weight_headroom_ratio, cfg.kv_cache_headroom_ratio, cfg.cuda_graphs,
            cfg.admit_skip) == (2048, 32, 32, 2.0, 0.90, 0.20, 0.20, False, 4)
    for bad in (dict(prefill_chunk_size=0), dict(max_batch_size=0), dict(max_queue_size=0),
                dict(batch_wait_ms=-1), dict(max_gpu_utilization=0), dict(max_gpu_utilization=1.5),
                dict(kv_cache_headroom_ratio=1.0), dict(weight_headroom_ratio=-0.1), dict(admit_skip=-1),
                dict(admit_skip=True),
                dict(dtype="float16"), dict(page_size=24)):
        with pytest.raises(ValueError):
            PylonConfig(**bad)
    monkeypatch.setenv("PYLON_PREFILL_CHUNK_SIZE", "512")
    monkeypatch.setenv("PYLON_CUDA_GRAPHS", "true")
    monkeypatch.setenv("PYLON_ADMIT_SKIP", "2")
    env = get_config()
    assert env.prefill_chunk_size == 512 and env.cuda_graphs is True and env.admit_skip == 2
    assert get_config(prefill_chunk_size=64).prefill_chunk_size == 64
    monkeypatch.setenv("PYLON_CUDA_GRAPHS", "yes")
    with pytest.raises(ValueError, match="PYLON_CUDA_GRAPHS = 'yes' cannot be read: expected true, false, 1 or 0"):
        get_config()
    monkeypatch.setenv("PYLON_CUDA_GRAPHS", "0")
    monkeypatch.setenv("PYLON_NUM_PAGES", "")
    monkeypatch.setenv("PYLON_MAX_BATCH_SIZE", "0")
    with pytest.raises(ValueError, match="max_batch_size = 0 is not allowed: it must be a whole number of at least 1"):
        get_config()
    assert get_config(max_batch_size=3).num_pages is None  # an argument wins over the variable
    with pytest.raises(TypeError, match="unknown option"):
        get_config(no_such_option=1)


def test_weights_must_fit_under_the_utilisation_limit():
    # /root/reference/src/pylon/kv/budget.py:49-68: weights times (1 + headroom) against
    # utilisation * total minus what is occupied
    import torch

    from pylon_amd.engine.runner import check_weights_fit, weight_bytes

    raw = dict(TINY_A)
    arch = resolve(raw)
    spec = arch.model_spec(arch.parse_config(raw))
    # embedding 256*64 (tied head), two layers of (64 + 64 + 16 + 16) norm weights,
    # qkv (64 + 2*32)*64, out 64*64, gate/up 2*128*64, down 64*128, and the final norm
    per_layer = 64 + 64 + 16 + 16 + 128 * 64 + 64 * 64 + 256 * 64 + 64 * 128
    norms = 2 * (64 + 64 + 16 + 16) + 64
    assert weight_bytes(spec, torch.bfloat16) == 2 * (256 * 64 + 2 * per_layer + 64 - norms) + 4 * norms
    total = 1000
    check_weights_fit(600, free=total, total=total, config=PylonConfig(), what="m")  # 720 <= 900
    with pytest.raises(RuntimeError, match="weights and headroom need 960 bytes; 900 bytes are available"):
        check_weights_fit(800, free=total, total=total, config=PylonConfig(), what="m")
    with pytest.raises(RuntimeError, match="720 bytes; 700 bytes"):
        check_weights_fit(600, free=800, total=total, config=PylonConfig(), what="m")  # 200 occupied


def test_stop_ids_come_from_generation_config_before_config(tmp_path):
    # /root/reference/src/pylon/model/tokenizer.py:24-38
    from pylon_amd.config import read_stop_token_ids

    (tmp_path / "config.json").write_text(json.dumps(dict(TINY_A, eos_token_id=7)))
    assert read_stop_token_ids(tmp_path) == (7,)
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [3, 9]}))
    assert read_stop_token_ids(tmp_path) == (3, 9)
    (tmp_path / "generation_config.json").write_text(json.dumps({"temperature": 0.6}))
    assert read_stop_token_ids(tmp_path) == (7,)
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    assert read_stop_token_ids(tmp_path) == ()


def test_pool_pages_follow_the_reference_budget():
    """/root/reference/src/pylon/kv/budget.py:70-113 with its own numbers: utilisation limit
    times total, minus what is occupied, minus free - free/(1 + ratio)."""
    from pylon_amd.config import PylonConfig
    from pylon_amd.engine.runner import pool_pages

    config = PylonConfig(page_size=16, max_batch_size=4, max_gpu_utilization=0.9, kv_cache_headroom_ratio=0.25)
    total, free = 1000_000, 600_000
    headroom = free - int(free / 1.25)  # 120,000
    budget = 900_000 - 400_000 - headroom  # 380,000
    assert pool_pages(free, total, 100, config, None) == budget // 1600
    assert pool_pages(free, total, 100, config, 64) == 4 * 4  # four requests of the longest length
    assert pool_pages(free, total, 100, config, 70) == 4 * 5
    import pytest

    with pytest.raises(RuntimeError, match="Not enough GPU memory"):
        pool_pages(free, total, 100_000, config, None)
    # the measured branch (:85-95): the headroom is the activations' peak times 1 + ratio
    from pylon_amd.engine.runner import cache_budget

    assert cache_budget(free, total, config, activation_bytes=40_000) == 900_000 - 400_000 - 50_000
    assert pool_pages(free, total, 100, config, None, activation_bytes=40_000) == 450_000 // 1600
    with pytest.raises(ValueError, match="non-negative"):
        cache_budget(free, total, config, activation_bytes=-1)
