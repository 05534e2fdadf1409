"""What a model does outside its layers is made of parts too.  Two toys defined here and
nowhere in the framework are registered, built and stepped without a change to its files: a
"stream" part that adds a learned vector per position to the embedded tokens, and a
"logits" part that bounds the logits by ``cap * tanh(logits / cap)``.  The toy architecture
is the tiny Qwen3 decoder with both; its logits are compared with a plain computation, whole,
in portions, and under graph replay.  Test fixtures, not models of anyone's."""
import dataclasses
from dataclasses import dataclass

import numpy as np
import pytest
import torch

from tests.helpers import TINY_B, random_tokens, read_folder
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu
POSITIONS = 160
CAP = 1.0


@dataclass(frozen=True)
class LearnedPositionsSpec:
    positions: int
    dim: int
    kind: str = "toy_learned_positions"


@dataclass(frozen=True)
class SoftCapSpec:
    cap: float
    kind: str = "toy_soft_cap"


def build_toys():
    from pylon_amd.config.registry import Architecture, WeightTarget
    from pylon_amd.models import qwen3
    from pylon_amd.parts.base import Part

    class LearnedPositions(Part):
        """resid_t += table[position_t], in the float32 residual stream."""

        def __init__(self, spec, *, dtype, device):
            super().__init__()
            self.add_param("table", (spec.positions, spec.dim), dtype, device)

        def forward(self, resid, ctx):
            return resid.add_(self.params["table"].index_select(0, ctx.positions).float())

    class SoftCap(Part):
        """logits <- cap * tanh(logits / cap), in place: a graph's replay leaves them where
        the step's caller reads them."""

        def __init__(self, spec, *, dtype, device):
            super().__init__()
            self.cap = spec.cap

        def forward(self, logits, ctx):
            return logits.div_(self.cap).tanh_().mul_(self.cap)

    def model_spec(cfg):
        return dataclasses.replace(
            qwen3.model_spec(cfg),
            stream_parts=(LearnedPositionsSpec(POSITIONS, cfg.hidden_size),),
            logit_parts=(SoftCapSpec(CAP),),
        )

    def weight_targets(cfg):
        targets = dict(qwen3.weight_targets(cfg))
        targets["model.position_table.weight"] = WeightTarget("stream.0.table", (POSITIONS, cfg.hidden_size))
        return targets

    def config_to_json(cfg):
        return dict(qwen3.config_to_json(cfg), architectures=["ToyOuterPartsForCausalLM"])

    arch = Architecture("ToyOuterPartsForCausalLM", qwen3.parse_config, model_spec, weight_targets, config_to_json)
    return arch, LearnedPositions, SoftCap


def plain_forward(weights, cfg, toks):
    w = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
    positions = np.arange(len(toks))
    x = w["model.embed_tokens.weight"][np.asarray(toks)] + w["model.position_table.weight"][positions]
    for layer in range(cfg["num_hidden_layers"]):
        x, _ = plain.block(x, w, layer, cfg, positions, None, None)
    x = plain.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    raw = x @ head.T
    return CAP * np.tanh(raw / CAP), raw


def close_rows(got, want, raw, tol):
    """Each row within ``tol`` of the largest logit before the cap: the cap contracts, so the
    bound that holds for the head's output holds after it."""
    excess = np.abs(got - want).max(axis=1) / np.abs(raw).max(axis=1)
    return bool((excess <= tol).all()), int(excess.argmax()), float(excess.max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_parts_before_the_first_layer_and_after_the_head(tmp_path, dtype):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.config import register_architecture, unregister_architecture
    from pylon_amd.engine import Runner, StepEntry
    from pylon_amd.parts import register_part, unregister_part
    from pylon_amd.weights import write_random_model

    arch, LearnedPositions, SoftCap = build_toys()
    register_architecture(arch)
    register_part("stream", "toy_learned_positions", LearnedPositions)
    register_part("logits", "toy_soft_cap", SoftCap)
    try:
        config = dict(TINY_B, architectures=["ToyOuterPartsForCausalLM"])
        # the weights of the other tests; the cap is well inside the logits, so a missing cap shows; the position table is
        # drawn like any other matrix, as large as the embedding it is added to
        folder = write_random_model(tmp_path / "toy", config, 9, dtype=dtype, std=0.08, norm_jitter=0.1)
        cfg, weights = read_folder(folder)
        assert "model.position_table.weight" in weights
        tol = 2e-5 if dtype == "float32" else 2e-2
        runner = Runner.from_folder(folder, dtype=dtype, page_size=16, num_pages=20, max_requests=3)
        reqs = {f"o{i}": random_tokens(cfg["vocab_size"], n, 500 + i) for i, n in enumerate((61, 18, 90))}
        want, raw = {}, {}
        for rid, toks in reqs.items():
            want[rid], raw[rid] = plain_forward(weights, cfg, toks)
        uncapped = plain.forward({k: v for k, v in weights.items() if "position_table" not in k}, cfg, reqs["o0"])
        assert np.abs(uncapped).max() > 2 * CAP and np.abs(want["o0"]).max() <= CAP
        assert np.abs(CAP * np.tanh(uncapped / CAP) - want["o0"]).max() > 0.1  # the table matters

        for rid, toks in reqs.items():  # whole
            seq = runner.open(rid)
            got = runner.step([StepEntry(seq, toks, list(range(len(toks))))]).cpu().numpy()
            runner.close(seq)
            assert close_rows(got, want[rid], raw[rid], tol)[0], (rid, close_rows(got, want[rid], raw[rid], tol))

        # portions of two requests side by side, then single tokens under graph replay
        runner.enable_graphs(2, max_tokens_per_request=128)
        seqs = {rid: runner.open(rid) for rid in ("o0", "o2")}
        got = {rid: [] for rid in seqs}
        cursor = {rid: 0 for rid in seqs}
        plan = [{"o0": 13, "o2": 2}, {"o0": 1, "o2": 40}, {"o0": 30, "o2": 1}, {"o0": 2, "o2": 31}]
        plan += [{"o0": 1, "o2": 1}] * 15
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
        assert runner.graphs.replays >= 14
        for rid in seqs:
            g = np.concatenate(got[rid])
            assert len(g) == cursor[rid] >= 61
            verdict = close_rows(g, want[rid][: len(g)], raw[rid][: len(g)], tol)
            assert verdict[0], (rid, verdict)
    finally:
        unregister_part("logits", "toy_soft_cap")
        unregister_part("stream", "toy_learned_positions")
        unregister_architecture("ToyOuterPartsForCausalLM")
