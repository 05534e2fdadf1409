"""A mixer with state of its own, defined here and nowhere in the framework, can be
registered, built into a model beside attention layers, loaded, and stepped: whole,
in portions, and mixed with other requests.  Nothing in ``pylon_amd`` is changed for it.

The toy is a leaky running sum: ``s_t = decay * s_{t-1} + h_t``, ``out_t = W s_t``; its
state is one vector per request, kept in the cache manager's state slots.  It is a test
fixture, not a model of anyone's."""
import dataclasses
from dataclasses import dataclass

import numpy as np
import pytest
import torch

from tests.helpers import TINY_A, random_tokens, read_folder
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@dataclass(frozen=True)
class LeakySumSpec:
    hidden_size: int
    decay: float
    kind: str = "leaky_sum"


def build_toy():
    from pylon_amd.config.registry import Architecture, WeightTarget
    from pylon_amd.models import qwen3
    from pylon_amd.parts.base import Part, StateRequirement

    class LeakySum(Part):
        def __init__(self, spec, *, dtype, device):
            super().__init__()
            self.spec, self.dtype = spec, dtype
            self.add_param("weight", (spec.hidden_size, spec.hidden_size), dtype, device)

        def cache_requirement(self):
            return StateRequirement((self.spec.hidden_size,), torch.float32)

        def forward(self, h, ctx, cache, stores):
            out = torch.empty_like(h)
            starts = ctx.row_start.cpu().tolist()
            slots = ctx.row_slots.cpu().tolist()
            for r in range(ctx.rows):
                s = cache.state[slots[r]].clone()
                for t in range(starts[r], starts[r + 1]):
                    s = self.spec.decay * s + h[t].float()
                    out[t] = (self.params["weight"].float() @ s).to(h.dtype)
                cache.state[slots[r]] = s
            return out

    def model_spec(cfg):
        spec = qwen3.model_spec(cfg)
        layers = list(spec.layers)
        layers[0] = dataclasses.replace(layers[0], mixer=LeakySumSpec(cfg.hidden_size, 0.75))
        return dataclasses.replace(spec, layers=tuple(layers))

    def weight_targets(cfg):
        targets = {k: v for k, v in qwen3.weight_targets(cfg).items()
                   if not k.startswith("model.layers.0.self_attn")}
        targets["model.layers.0.leaky.weight"] = WeightTarget(
            "layers.0.mixer.weight", (cfg.hidden_size, cfg.hidden_size))
        return targets

    def config_to_json(cfg):
        return dict(qwen3.config_to_json(cfg), architectures=["ToyLeakyForCausalLM"])

    arch = Architecture("ToyLeakyForCausalLM", qwen3.parse_config, model_spec, weight_targets, config_to_json)
    return arch, LeakySum


def plain_toy_forward(weights, cfg, toks):
    """Layer 0: leaky sum in place of attention; layer 1: the plain Qwen3 block."""
    w = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
    x = w["model.embed_tokens.weight"][np.asarray(toks)]
    eps = cfg["rms_norm_eps"]
    h = plain.rms_norm(x, w["model.layers.0.input_layernorm.weight"], eps)
    s = np.zeros(cfg["hidden_size"])
    mixed = np.zeros_like(h)
    for t in range(len(toks)):
        s = 0.75 * s + h[t]
        mixed[t] = w["model.layers.0.leaky.weight"] @ s
    x = x + mixed
    h = plain.rms_norm(x, w["model.layers.0.post_attention_layernorm.weight"], eps)
    x = x + plain.gated_feed_forward(h, w["model.layers.0.mlp.gate_proj.weight"],
                                     w["model.layers.0.mlp.up_proj.weight"], w["model.layers.0.mlp.down_proj.weight"])
    x, _ = plain.block(x, w, 1, cfg, np.arange(len(toks)))
    x = plain.rms_norm(x, w["model.norm.weight"], eps)
    return x @ w["model.embed_tokens.weight"].T


def test_a_stateful_toy_mixer_registers_builds_and_steps(tmp_path):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.config import register_architecture, unregister_architecture
    from pylon_amd.engine import Runner, StepEntry
    from pylon_amd.parts import register_part, unregister_part
    from pylon_amd.weights import write_random_model

    arch, LeakySum = build_toy()
    register_architecture(arch)
    register_part("mixer", "leaky_sum", LeakySum)
    try:
        config = dict(TINY_A, architectures=["ToyLeakyForCausalLM"])
        folder = write_random_model(tmp_path / "toy", config, 3, dtype="float32", std=0.08, norm_jitter=0.1)
        cfg, weights = read_folder(folder)
        runner = Runner.from_folder(folder, dtype="float32", page_size=16, num_pages=12, max_requests=3)
        # run 0 keeps a state vector per request, run 1 keeps keys and values
        assert list(runner.manager.slots.tensors) == [0] and runner.manager.group_of == {1: 0}
        reqs = {f"t{i}": random_tokens(cfg["vocab_size"], n, 200 + i) for i, n in enumerate((40, 23, 57))}
        want = {rid: plain_toy_forward(weights, cfg, toks) for rid, toks in reqs.items()}
        # whole
        for rid, toks in reqs.items():
            seq = runner.open(rid)
            got = runner.step([StepEntry(seq, toks, list(range(len(toks))))]).cpu().numpy()
            runner.close(seq)
            assert np.abs(got - want[rid]).max() <= 2e-5 * np.abs(want[rid]).max(), rid
        # mixed: portions of some beside single tokens of others; state slots are reused
        live = {rid: runner.open(rid) for rid in ("t0", "t1")}
        pos = {rid: 0 for rid in reqs}
        got = {rid: [] for rid in reqs}
        plan = [{"t0": 7, "t1": 1}, {"t0": 1, "t1": 9}, {"t1": 13}, {"t0": 32}, {"t1": 0, "t2": 5},
                {"t2": 1}, {"t2": 30}, {"t2": 21}]
        for step in plan:
            entries = []
            for rid, size in step.items():
                if size == 0:
                    runner.close(live.pop(rid))
                    continue
                if rid not in live:
                    live[rid] = runner.open(rid)
                chunk = reqs[rid][pos[rid]: pos[rid] + size]
                entries.append((rid, StepEntry(live[rid], chunk, list(range(len(chunk))))))
                pos[rid] += len(chunk)
            logits = runner.step([e for _, e in entries]).cpu().numpy()
            cursor = 0
            for rid, e in entries:
                got[rid].append(logits[cursor: cursor + len(e.tokens)])
                cursor += len(e.tokens)
        assert live["t2"].slot == 1  # t1's slot, handed out again and cleared
        for rid in reqs:
            g = np.concatenate(got[rid])
            assert np.abs(g - want[rid][: len(g)]).max() <= 2e-5 * np.abs(want[rid]).max(), rid
        assert pos == {"t0": 40, "t1": 23, "t2": 57}
        for seq in list(live.values()):
            runner.close(seq)

        # a step that fails in the second layer, after the toy mixer has overwritten its state:
        # pages, lengths and the state are as before it, and the request goes on correctly
        toks = reqs["t0"]
        seq = runner.open("again")
        head = runner.step([StepEntry(seq, toks[:10], list(range(10)))]).cpu().numpy()
        state_before = runner.manager.slots.tensors[0][seq.slot].clone()
        free_before = runner.manager.free_pages
        second = runner.model.blocks[1]
        intact = second.forward

        def broken(*args, **kwargs):
            raise RuntimeError("the second layer failed")

        second.forward = broken
        try:
            with pytest.raises(RuntimeError, match="second layer failed"):
                runner.step([StepEntry(seq, toks[10:30], [])])
        finally:
            second.forward = intact
        assert seq.length == 10 and runner.manager.free_pages == free_before
        assert torch.equal(runner.manager.slots.tensors[0][seq.slot], state_before)
        runner.manager.check()
        rest = runner.step([StepEntry(seq, toks[10:], list(range(len(toks) - 10)))]).cpu().numpy()
        runner.close(seq)
        got_again = np.concatenate([head, rest])
        assert np.abs(got_again - want["t0"]).max() <= 2e-5 * np.abs(want["t0"]).max()

        # start-up takes the state's bytes off the budget before it counts pages
        from pylon_amd.config import PylonConfig

        sized = Runner.from_config(PylonConfig(model_path=str(folder), dtype="float32", page_size=16,
                                               max_batch_size=3))
        assert sized.pool_sizing["state_bytes"] == 3 * cfg["hidden_size"] * 4
        assert sized.pool_sizing["bytes_per_token"] == 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * 4
        assert sized.manager.num_pages == 3 * (cfg["max_position_embeddings"] // 16)
    finally:
        unregister_part("mixer", "leaky_sum")
        unregister_architecture("ToyLeakyForCausalLM")
