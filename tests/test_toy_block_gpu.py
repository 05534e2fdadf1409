"""Another norm and another arrangement of a layer's parts, defined here and nowhere in the
framework: a centred norm with a bias (mean removed, variance normalised), and a block in
which the mixer and the feed-forward read the same normed input and both add to the
residual, ``x = x + mixer(norm(x)) + feed_forward(norm(x))``.  They are registered, built
into a model beside the ordinary parts, loaded from a model folder written by the
random-weights mode, and stepped whole, in portions and under graph replay.  Nothing in
``pylon_amd`` is changed for them.  Test fixtures, not models of anyone's."""
import dataclasses
from dataclasses import dataclass

import numpy as np
import pytest
import torch

from tests.helpers import TINY_C, random_tokens, read_folder, rows_within
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu


@dataclass(frozen=True)
class CentredNormSpec:
    dim: int
    eps: float
    kind: str = "toy_centred"


def build_toys():
    from pylon_amd.config.registry import Architecture, WeightTarget
    from pylon_amd.models import qwen3
    from pylon_amd.parts.base import Part, summed
    from pylon_amd.parts.registry import build_part

    class CentredNorm(Part):
        """y = (x - mean) / sqrt(var + eps) * weight + bias, in float32, rounded once."""

        def __init__(self, spec, *, dtype, device):
            super().__init__()
            self.spec, self.dtype = spec, dtype
            self.add_param("weight", (spec.dim,), torch.float32, device, role="vector")
            self.add_param("bias", (spec.dim,), torch.float32, device, role="vector")

        def forward(self, x):
            x = x.float()
            centred = x - x.mean(dim=-1, keepdim=True)
            y = centred / torch.sqrt(centred.pow(2).mean(dim=-1, keepdim=True) + self.spec.eps)
            return (y * self.params["weight"] + self.params["bias"]).to(self.dtype)

        def add_forward(self, resid, delta, *, row_idx=None):
            d = summed(delta)
            if row_idx is not None:  # only these rows, and the residual stays
                rows = resid.index_select(0, row_idx.long())
                return self.forward(rows if d is None else rows + d.index_select(0, row_idx.long()))
            if d is not None:
                resid.add_(d)
            return self.forward(resid)

    class ParallelBlock(Part):
        """One norm; the mixer and the feed-forward both read it; their outputs go on together."""

        def __init__(self, spec, *, dtype, device):
            super().__init__()
            kw = dict(dtype=dtype, device=device)
            self.norm = self.add_child("mixer_norm", build_part("norm", spec.mixer_norm, **kw))
            self.mixer = self.add_child("mixer", build_part("mixer", spec.mixer, **kw))
            self.feed_forward = self.add_child("feed_forward", build_part("feed_forward", spec.feed_forward, **kw))

        def cache_requirement(self):
            return self.mixer.cache_requirement()

        def forward(self, resid, delta, ctx, cache, stores):
            h = self.norm.add_forward(resid, delta)
            return resid, summed(self.mixer.forward(h, ctx, cache, stores)) + summed(self.feed_forward.forward(h, ctx))

    def model_spec(cfg):
        spec = qwen3.model_spec(cfg)
        norm = CentredNormSpec(cfg.hidden_size, cfg.rms_norm_eps)
        layers = tuple(dataclasses.replace(layer, mixer_norm=norm, arrangement="toy_parallel") for layer in spec.layers)
        return dataclasses.replace(spec, layers=layers)

    def weight_targets(cfg):
        targets = {k: v for k, v in qwen3.weight_targets(cfg).items() if "post_attention_layernorm" not in k}
        for layer in range(cfg.num_hidden_layers):
            targets[f"model.layers.{layer}.input_layernorm.bias"] = WeightTarget(
                f"layers.{layer}.mixer_norm.bias", (cfg.hidden_size,), role="vector")
        return targets

    def config_to_json(cfg):
        return dict(qwen3.config_to_json(cfg), architectures=["ToyParallelForCausalLM"])

    arch = Architecture("ToyParallelForCausalLM", qwen3.parse_config, model_spec, weight_targets, config_to_json)
    return arch, CentredNorm, ParallelBlock


def plain_forward(weights, cfg, toks):
    w = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
    positions = np.arange(len(toks))
    x = w["model.embed_tokens.weight"][np.asarray(toks)]
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}"
        centred = x - x.mean(axis=-1, keepdims=True)
        h = centred / np.sqrt((centred ** 2).mean(axis=-1, keepdims=True) + cfg["rms_norm_eps"])
        h = h * w[f"{p}.input_layernorm.weight"] + w[f"{p}.input_layernorm.bias"]
        mixed, _ = plain.attention_half(h, w, p, cfg, positions)
        x = x + mixed + plain.gated_feed_forward(h, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                                                 w[f"{p}.mlp.down_proj.weight"])
    x = plain.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return x @ head.T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_another_norm_and_another_arrangement_of_a_layer(tmp_path, dtype):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.config import register_architecture, unregister_architecture
    from pylon_amd.engine import Runner, StepEntry
    from pylon_amd.parts import register_part, unregister_part
    from pylon_amd.weights import write_random_model

    arch, CentredNorm, ParallelBlock = build_toys()
    register_architecture(arch)
    register_part("norm", "toy_centred", CentredNorm)
    register_part("block", "toy_parallel", ParallelBlock)
    try:
        config = dict(TINY_C, architectures=["ToyParallelForCausalLM"])
        folder = write_random_model(tmp_path / "toy", config, 13, dtype=dtype, std=0.08, norm_jitter=0.1)
        cfg, weights = read_folder(folder)
        assert "model.layers.1.input_layernorm.bias" in weights
        assert "model.layers.0.post_attention_layernorm.weight" not in weights
        tol = 2e-5 if dtype == "float32" else 2e-2
        runner = Runner.from_folder(folder, dtype=dtype, page_size=16, num_pages=20, max_requests=3)
        reqs = {f"p{i}": random_tokens(cfg["vocab_size"], n, 700 + i) for i, n in enumerate((57, 19, 84))}
        want = {rid: plain_forward(weights, cfg, toks) for rid, toks in reqs.items()}
        # the ordinary arrangement of the same weights gives other logits: the toys are in use
        ordinary = plain.forward(
            {k: v for k, v in weights.items() if not k.endswith("input_layernorm.bias")}
            | {f"model.layers.{i}.post_attention_layernorm.weight": weights[f"model.layers.{i}.input_layernorm.weight"]
               for i in range(cfg["num_hidden_layers"])}, cfg, reqs["p1"])
        assert np.abs(ordinary - want["p1"]).max() > 1e-2

        for rid, toks in reqs.items():  # whole
            seq = runner.open(rid)
            got = runner.step([StepEntry(seq, toks, list(range(len(toks))))]).cpu().numpy()
            runner.close(seq)
            assert rows_within(got, want[rid], tol)[0], (rid, rows_within(got, want[rid], tol))

        # portions of two requests side by side, then single tokens under graph replay
        runner.enable_graphs(2, max_tokens_per_request=128)
        seqs = {rid: runner.open(rid) for rid in ("p0", "p2")}
        got = {rid: [] for rid in seqs}
        cursor = {rid: 0 for rid in seqs}
        plan = [{"p0": 11, "p2": 2}, {"p0": 1, "p2": 37}, {"p0": 29, "p2": 1}, {"p0": 2, "p2": 30}]
        plan += [{"p0": 1, "p2": 1}] * 14
        for sizes in plan:
            entries = []
            for rid, n in sizes.items():
                chunk = reqs[rid][cursor[rid]: cursor[rid] + n]
                cursor[rid] += len(chunk)
                entries.append(StepEntry(seqs[rid], chunk, list(range(len(chunk)))))
            logits = runner.step(entries).cpu().numpy()
            at = 0
            for rid, e in zip(sizes, entries):
                got[rid].append(logits[at: at + len(e.tokens)])
                at += len(e.tokens)
        assert runner.graphs.replays >= 13
        for rid in seqs:
            g = np.concatenate(got[rid])
            assert len(g) == cursor[rid] >= 57
            verdict = rows_within(g, want[rid][: len(g)], tol)
            assert verdict[0], (rid, verdict)
    finally:
        unregister_part("block", "toy_parallel")
        unregister_part("norm", "toy_centred")
        unregister_architecture("ToyParallelForCausalLM")
