"""Parts defined here and nowhere in the framework can take the place of a layer's
feed-forward and of its position encoding: a feed-forward that routes each token to one of
three small experts, and a rotary encoding with frequencies of its own over half of every
head.  They are registered, built into a model beside the ordinary parts, loaded from a
model folder written by the random-weights mode, and stepped whole and in portions.
Nothing in ``pylon_amd`` is changed for them.  They are test fixtures, not models of
anyone's."""
import dataclasses
import math
from dataclasses import dataclass

import numpy as np
import pytest
import torch

from tests.helpers import TINY_C, random_tokens, read_folder
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu
EXPERTS = 3


@dataclass(frozen=True)
class RoutedSpec:
    hidden_size: int
    experts: int
    kind: str = "toy_routed"


@dataclass(frozen=True)
class HarmonicSpec:
    rotary_dim: int
    base: float
    max_positions: int = 0
    kind: str = "toy_harmonic"


def build_toys():
    from pylon_amd.config.registry import Architecture, WeightTarget
    from pylon_amd.kernels import ops
    from pylon_amd.models import qwen3
    from pylon_amd.parts.base import Part

    class Routed(Part):
        """out_t = p_t[e] * W_e h_t for the expert e with the largest router probability."""

        def __init__(self, spec, *, dtype, device):
            super().__init__()
            self.spec, self.dtype = spec, dtype
            self.add_param("router", (spec.experts, spec.hidden_size), torch.float32, device)
            self.add_param("experts", (spec.experts * spec.hidden_size, spec.hidden_size), dtype, device)

        def forward(self, h, ctx):
            hidden = self.spec.hidden_size
            logits = ops.linear(h.float(), self.params["router"], out_dtype=torch.float32)  # routing in 32-bit
            probs = torch.softmax(logits, dim=-1)
            weight, choice = probs.max(dim=-1)
            out = torch.zeros_like(h)
            for e in range(self.spec.experts):
                rows = torch.nonzero(choice == e).flatten()
                if rows.numel():
                    w = self.params["experts"][e * hidden: (e + 1) * hidden]
                    y = ops.linear(h[rows].contiguous(), w, out_dtype=torch.float32)
                    out[rows] = (y * weight[rows, None]).to(h.dtype)
            return out

    class Harmonic(Part):
        """Frequencies base / (i + 1) over the first rotary_dim elements of a head."""

        def __init__(self, spec, *, dtype, device):
            super().__init__()
            self.spec = spec
            i = torch.arange(spec.rotary_dim // 2, dtype=torch.float32)
            self.inv_freq = (torch.tensor(spec.base, dtype=torch.float32) / (i + 1)).to(device)

        def rotary(self):
            return self.inv_freq, self.spec.rotary_dim

    def model_spec(cfg):
        spec = qwen3.model_spec(cfg)
        layers = list(spec.layers)
        mixer = dataclasses.replace(layers[0].mixer, position=HarmonicSpec(cfg.head_dim // 2, 0.37))
        layers[0] = dataclasses.replace(layers[0], mixer=mixer)
        layers[1] = dataclasses.replace(layers[1], feed_forward=RoutedSpec(cfg.hidden_size, EXPERTS))
        return dataclasses.replace(spec, layers=tuple(layers))

    def weight_targets(cfg):
        targets = {k: v for k, v in qwen3.weight_targets(cfg).items() if not k.startswith("model.layers.1.mlp")}
        h = cfg.hidden_size
        targets["model.layers.1.router.weight"] = WeightTarget("layers.1.feed_forward.router", (EXPERTS, h))
        for e in range(EXPERTS):
            targets[f"model.layers.1.experts.{e}.weight"] = WeightTarget(
                "layers.1.feed_forward.experts", (h, h), row_start=e * h)
        return targets

    def config_to_json(cfg):
        return dict(qwen3.config_to_json(cfg), architectures=["ToyRoutedForCausalLM"])

    arch = Architecture("ToyRoutedForCausalLM", qwen3.parse_config, model_spec, weight_targets, config_to_json)
    return arch, Routed, Harmonic


def plain_forward(weights, cfg, toks):
    """Layer 0: attention with the harmonic half-head rotation; layer 1: attention as in
    Qwen3, then the routed feed-forward."""
    w = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, tokens = cfg["rms_norm_eps"], len(toks)
    positions = np.arange(tokens)
    x = w["model.embed_tokens.weight"][np.asarray(toks)]

    # layer 0, attention half with the toy rotation
    p = "model.layers.0"
    h = plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], eps)
    rot = hd // 2
    inv = (np.float32(0.37) / (np.arange(rot // 2, dtype=np.float32) + 1)).astype(np.float32)
    angles = (positions.astype(np.float32)[:, None] * inv[None, :]).astype(np.float64)  # float32 products
    cos, sin = np.cos(angles), np.sin(angles)

    def rotate(v):  # v: [heads, tokens, hd]; element i pairs with i + rot/2, the rest stays
        out = v.copy()
        a, b = v[..., : rot // 2], v[..., rot // 2: rot]
        out[..., : rot // 2] = a * cos - b * sin
        out[..., rot // 2: rot] = b * cos + a * sin
        return out

    def heads(name, n):
        return (h @ w[f"{p}.self_attn.{name}_proj.weight"].T).reshape(tokens, n, hd).transpose(1, 0, 2)

    q = rotate(plain.rms_norm(heads("q", nh), w[f"{p}.self_attn.q_norm.weight"], eps))
    k = rotate(plain.rms_norm(heads("k", nkv), w[f"{p}.self_attn.k_norm.weight"], eps))
    attended = plain.causal_attention(q, k, heads("v", nkv), 1.0 / math.sqrt(hd))
    x = x + attended.transpose(1, 0, 2).reshape(tokens, nh * hd) @ w[f"{p}.self_attn.o_proj.weight"].T
    h = plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps)
    x = x + plain.gated_feed_forward(h, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                                     w[f"{p}.mlp.down_proj.weight"])

    # layer 1, ordinary attention, then the routed feed-forward
    p = "model.layers.1"
    a, _ = plain.attention_half(plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], eps), w, p, cfg, positions)
    x = x + a
    h = plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps)
    probs = plain.softmax(h @ w[f"{p}.router.weight"].T)
    choice = probs.argmax(axis=-1)
    routed = np.stack([probs[t, choice[t]] * (w[f"{p}.experts.{choice[t]}.weight"] @ h[t]) for t in range(tokens)])
    x = x + routed
    x = plain.rms_norm(x, w["model.norm.weight"], eps)
    return x @ w["lm_head.weight"].T, choice


def test_a_routed_feed_forward_and_another_position_encoding_take_their_places(tmp_path):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.config import register_architecture, unregister_architecture
    from pylon_amd.engine import Runner, StepEntry
    from pylon_amd.parts import register_part, unregister_part
    from pylon_amd.weights import write_random_model

    arch, Routed, Harmonic = build_toys()
    register_architecture(arch)
    register_part("feed_forward", "toy_routed", Routed)
    register_part("position", "toy_harmonic", Harmonic)
    try:
        config = dict(TINY_C, architectures=["ToyRoutedForCausalLM"])
        folder = write_random_model(tmp_path / "toy", config, 5, dtype="float32", std=0.08, norm_jitter=0.1)
        cfg, weights = read_folder(folder)
        assert "model.layers.1.experts.2.weight" in weights and "model.layers.1.mlp.down_proj.weight" not in weights
        runner = Runner.from_folder(folder, dtype="float32", page_size=16, num_pages=16, max_requests=3)
        reqs = {f"t{i}": random_tokens(cfg["vocab_size"], n, 300 + i) for i, n in enumerate((50, 21, 77))}
        want, used = {}, set()
        for rid, toks in reqs.items():
            want[rid], choice = plain_forward(weights, cfg, toks)
            used |= set(choice.tolist())
        assert used == set(range(EXPERTS))  # every expert is taken by some token
        for rid, toks in reqs.items():  # whole
            seq = runner.open(rid)
            got = runner.step([StepEntry(seq, toks, list(range(len(toks))))]).cpu().numpy()
            runner.close(seq)
            assert np.abs(got - want[rid]).max() <= 2e-5 * np.abs(want[rid]).max(), rid
        # portions of two requests side by side, then single tokens
        seqs = {rid: runner.open(rid) for rid in ("t0", "t2")}
        got = {rid: [] for rid in seqs}
        cursor = {rid: 0 for rid in seqs}
        for sizes in ({"t0": 13, "t2": 2}, {"t0": 1, "t2": 40}, {"t0": 30, "t2": 1}, {"t0": 6, "t2": 34}):
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
        for rid in seqs:
            g = np.concatenate(got[rid])
            assert len(g) == len(reqs[rid])
            assert np.abs(g - want[rid]).max() <= 2e-5 * np.abs(want[rid]).max(), rid
        # the same weights under the ordinary rotation give other logits: the toy encoding is in use
        ordinary = plain.forward({k: v for k, v in weights.items() if "router" not in k and "experts" not in k}
                                 | {f"model.layers.1.mlp.{n}_proj.weight": weights["model.layers.0.mlp." + n + "_proj.weight"]
                                    for n in ("gate", "up", "down")}, cfg, reqs["t1"])
        assert np.abs(ordinary - want["t1"]).max() > 1e-3
    finally:
        unregister_part("position", "toy_harmonic")
        unregister_part("feed_forward", "toy_routed")
        unregister_architecture("ToyRoutedForCausalLM")
