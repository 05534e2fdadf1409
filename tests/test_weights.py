"""The weight loader and the random-weights mode (CPU tensors; no kernels involved)."""
import json

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

from pylon_amd.config import load_model_config
from pylon_amd.engine.model import Model
from pylon_amd.weights import WeightsError, load_weights, write_random_model
from tests.helpers import TINY_A, TINY_B, make_model_folder


def _load(folder, dtype):
    arch, cfg = load_model_config(folder)
    model = Model(arch.model_spec(cfg), dtype=dtype, device="cpu")
    load_weights(model, arch, cfg, folder)
    return model


def test_random_mode_is_a_function_of_config_and_seed(tmp_path):
    a = write_random_model(tmp_path / "a", TINY_B, 7, dtype="float32", norm_jitter=0.2)
    b = write_random_model(tmp_path / "b", TINY_B, 7, dtype="float32", norm_jitter=0.2)
    c = write_random_model(tmp_path / "c", TINY_B, 8, dtype="float32", norm_jitter=0.2)
    ta, tb, tc = (load_file(str(p / "model.safetensors")) for p in (a, b, c))
    assert set(ta) == set(tb) and all(torch.equal(ta[k], tb[k]) for k in ta)
    assert not torch.equal(ta["model.embed_tokens.weight"], tc["model.embed_tokens.weight"])
    assert json.loads((a / "config.json").read_text())["architectures"] == ["Qwen3ForCausalLM"]
    assert abs(float(ta["model.layers.0.mlp.down_proj.weight"].std()) - 0.02) < 2e-3
    assert not torch.allclose(ta["model.norm.weight"], torch.ones(96))  # drawn norm weights
    assert "lm_head.weight" in ta  # untied
    tied = load_file(str(write_random_model(tmp_path / "d", TINY_A, 1) / "model.safetensors"))
    assert "lm_head.weight" not in tied and tied["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert torch.equal(tied["model.norm.weight"].float(), torch.ones(64))


def test_q_k_v_and_gate_up_land_in_their_row_ranges(tmp_path):
    # /root/reference/tests/test_loader.py:33-77 pins the same order
    folder = make_model_folder(tmp_path, "B", dtype="float32")
    raw = load_file(str(folder / "model.safetensors"))
    model = _load(folder, torch.float32)
    mixer = model.blocks[1].mixer
    q, kv = 6 * 32, 1 * 32
    qkv = mixer.params["qkv"]
    assert qkv.shape == (q + 2 * kv, 96)
    assert torch.equal(qkv[:q], raw["model.layers.1.self_attn.q_proj.weight"])
    assert torch.equal(qkv[q:q + kv], raw["model.layers.1.self_attn.k_proj.weight"])
    assert torch.equal(qkv[q + kv:], raw["model.layers.1.self_attn.v_proj.weight"])
    ff = model.blocks[2].feed_forward
    assert torch.equal(ff.params["gate_up"][:320], raw["model.layers.2.mlp.gate_proj.weight"])
    assert torch.equal(ff.params["gate_up"][320:], raw["model.layers.2.mlp.up_proj.weight"])
    assert torch.equal(ff.params["down"], raw["model.layers.2.mlp.down_proj.weight"])
    assert torch.equal(model.params["lm_head"], raw["lm_head.weight"])
    assert torch.equal(mixer.params["k_norm"], raw["model.layers.1.self_attn.k_norm.weight"])
    assert torch.equal(model.final_norm.params["weight"], raw["model.norm.weight"])


def test_element_types_follow_what_is_stored(tmp_path):
    folder = make_model_folder(tmp_path, "A", dtype="bfloat16")
    model = _load(folder, torch.bfloat16)
    assert model.params["embed"].dtype == torch.bfloat16
    assert model.blocks[0].mixer.params["qkv"].dtype == torch.bfloat16
    assert model.blocks[0].mixer_norm.params["weight"].dtype == torch.float32  # vectors stay float32
    assert model.blocks[0].mixer.params["q_norm"].dtype == torch.float32
    # a tensor stored in 32-bit stays so, also in a bfloat16 model
    raw = load_file(str(folder / "model.safetensors"))
    raw["model.layers.1.mlp.down_proj.weight"] = raw["model.layers.1.mlp.down_proj.weight"].float() + 1e-4
    save_file(raw, str(folder / "model.safetensors"))
    model = _load(folder, torch.bfloat16)
    down = model.blocks[1].feed_forward.params["down"]
    assert down.dtype == torch.float32 and torch.equal(down, raw["model.layers.1.mlp.down_proj.weight"])
    assert model.blocks[0].feed_forward.params["down"].dtype == torch.bfloat16
    # a float32 model takes everything as float32
    assert _load(folder, torch.float32).params["embed"].dtype == torch.float32
    # start-up counts the weights with the types they will have, from the headers alone
    from pylon_amd.engine.runner import weight_bytes
    from pylon_amd.weights.loader import stored_param_dtypes

    arch, cfg = load_model_config(folder)
    spec = arch.model_spec(cfg)
    meta = Model(spec, dtype=torch.bfloat16, device="meta")
    dtypes = stored_param_dtypes(meta, arch, cfg, folder)
    assert dtypes["layers.1.feed_forward.down"] == torch.float32
    assert dtypes["layers.0.feed_forward.down"] == torch.bfloat16 and dtypes["final_norm.weight"] == torch.float32
    extra = 2 * down.numel()  # two more bytes for each of its elements
    assert weight_bytes(spec, torch.bfloat16, dtypes) == weight_bytes(spec, torch.bfloat16) + extra
    real = sum(o.params[n].numel() * o.params[n].element_size() for _, o, n in model.named_params())
    assert weight_bytes(spec, torch.bfloat16, dtypes) == real


def test_matrices_kept_in_32_bit_are_reported(tmp_path, caplog):
    folder = make_model_folder(tmp_path, "A", dtype="float32")
    with caplog.at_level("WARNING", logger="pylon"):
        model = _load(folder, torch.bfloat16)
    assert model.params["embed"].dtype == torch.float32
    assert "weights_kept_32bit" in caplog.text and "twice the memory" in caplog.text
    caplog.clear()
    with caplog.at_level("WARNING", logger="pylon"):
        _load(folder, torch.float32)
        _load(make_model_folder(tmp_path, "A", dtype="bfloat16"), torch.bfloat16)
    assert "weights_kept_32bit" not in caplog.text


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = make_model_folder(tmp_path, "A", dtype="float32")
    raw = load_file(str(folder / "model.safetensors"))
    del raw["model.layers.0.self_attn.k_proj.weight"]
    del raw["model.norm.weight"]
    raw["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    raw["model.layers.1.mlp.up_proj.weight"] = torch.zeros(64, 128)  # transposed
    raw["model.layers.1.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    save_file(raw, str(folder / "model.safetensors"))
    with pytest.raises(WeightsError) as info:
        _load(folder, torch.float32)
    err = info.value
    assert err.missing == ["model.layers.0.self_attn.k_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert len(err.wrong) == 2
    text = str(err)
    assert "expected shape (128, 64), got (64, 128)" in text and "stored as I32" in text
    assert "model.norm.weight" in text and "rotary_emb" in text


def test_a_tensor_the_architecture_does_not_know_is_skipped(tmp_path, caplog):
    # /root/reference/src/pylon/model/weights.py:22-25 passes over names it has no target for
    folder = make_model_folder(tmp_path, "A", dtype="float32")
    raw = load_file(str(folder / "model.safetensors"))
    raw["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(raw, str(folder / "model.safetensors"))
    arch, cfg = load_model_config(folder)
    model = Model(arch.model_spec(cfg), dtype=torch.float32, device="cpu")
    with caplog.at_level("WARNING", logger="pylon"):
        skipped = load_weights(model, arch, cfg, folder)
    assert skipped == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert "rotary_emb.inv_freq" in caplog.text
    assert torch.equal(model.params["embed"], raw["model.embed_tokens.weight"])
    with pytest.raises(WeightsError) as info:  # on request it is an error of its own
        load_weights(Model(arch.model_spec(cfg), dtype=torch.float32, device="cpu"), arch, cfg, folder,
                     strict=True)
    assert info.value.unexpected == skipped and not info.value.missing


def test_tied_head_is_optional_and_untied_head_is_required(tmp_path):
    folder = make_model_folder(tmp_path, "A", dtype="float32")
    raw = load_file(str(folder / "model.safetensors"))
    raw["lm_head.weight"] = raw["model.embed_tokens.weight"].clone()
    save_file(raw, str(folder / "model.safetensors"))
    model = _load(folder, torch.float32)  # a tied checkpoint that carries the head loads
    assert torch.equal(model.head_weight, raw["model.embed_tokens.weight"])
    folder_b = make_model_folder(tmp_path, "B", dtype="float32")
    raw = load_file(str(folder_b / "model.safetensors"))
    del raw["lm_head.weight"]
    save_file(raw, str(folder_b / "model.safetensors"))
    with pytest.raises(WeightsError, match="lm_head.weight"):
        _load(folder_b, torch.float32)


def test_sharded_folder_and_missing_file(tmp_path):
    folder = make_model_folder(tmp_path, "A", dtype="float32")
    raw = load_file(str(folder / "model.safetensors"))
    names = sorted(raw)
    half = len(names) // 2
    save_file({n: raw[n] for n in names[:half]}, str(folder / "model-00001-of-00002.safetensors"))
    save_file({n: raw[n] for n in names[half:]}, str(folder / "model-00002-of-00002.safetensors"))
    (folder / "model.safetensors").unlink()
    weight_map = {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                  for i, n in enumerate(names)}
    (folder / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    model = _load(folder, torch.float32)
    assert torch.equal(model.params["embed"], raw["model.embed_tokens.weight"])
    (folder / "model-00002-of-00002.safetensors").unlink()
    with pytest.raises(FileNotFoundError):
        _load(folder, torch.float32)


def test_filling_a_model_in_place_follows_the_folder_rule(tmp_path):
    # on the CPU the two ways of the random-weights mode give the same numbers
    from pylon_amd.weights import fill_random_model

    folder = write_random_model(tmp_path / "m", TINY_B, 5, dtype="float32", norm_jitter=0.2)
    loaded = _load(folder, torch.float32)
    arch, cfg = load_model_config(folder)
    filled = Model(arch.model_spec(cfg), dtype=torch.float32, device="cpu")
    for _, owner, name in filled.named_params():
        owner.params[name].fill_(float("nan"))
    fill_random_model(filled, arch, cfg, 5, norm_jitter=0.2)
    for (path, a_owner, a_name), (_, b_owner, b_name) in zip(loaded.named_params(), filled.named_params()):
        assert torch.equal(a_owner.params[a_name], b_owner.params[b_name]), path
