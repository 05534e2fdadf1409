"""Configurations drawn at random over everything config.json allows: head sizes in steps of
16 from 16 to 512, any number of heads and groups, widths that are multiples of 2, 4 or 8 only,
vocabularies and feed-forward widths that are no power of two, tied and untied heads, page
sizes from 16 to 256.  Each is run whole, then token by token, then two requests side by
side in portions, in float32 and bfloat16, against the plain model: a kernel meets a size it
was not written at and must either take it or refuse it, never be wrong."""
import numpy as np
import pytest
import torch

from tests import traces
from tests.helpers import _qwen3, make_model_folder, random_tokens, read_folder, rows_within
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu
BOUND = {"float32": 2e-5, "bfloat16": 2e-2}


# Corners the draws may miss: a width that is a multiple of 2 only with the largest head size
# and seven query heads to a key/value head; a width that is a multiple of 4 only with the
# smallest head size and sixteen query heads to one key/value head; a width from which on a
# bfloat16 model keeps the rows of its gate/up matrix apart in memory.
CORNERS = {
    "wide": (dict(num_hidden_layers=1, hidden_size=1032, num_attention_heads=6, num_key_value_heads=3, head_dim=64,
                  intermediate_size=2050, vocab_size=333, rope_theta=1e6, rms_norm_eps=1e-6,
                  tie_word_embeddings=True, max_position_embeddings=512), 32, (7, 90, 150)),
    "narrow": (dict(num_hidden_layers=2, hidden_size=50, num_attention_heads=7, num_key_value_heads=1, head_dim=512,
                    intermediate_size=34, vocab_size=131, rope_theta=12345.0, rms_norm_eps=3e-5,
                    tie_word_embeddings=True, max_position_embeddings=512), 16, (3, 70, 210)),
    "many_heads": (dict(num_hidden_layers=1, hidden_size=108, num_attention_heads=32, num_key_value_heads=2, head_dim=16,
                        intermediate_size=250, vocab_size=1021, rope_theta=2.5e6, rms_norm_eps=1e-6,
                        tie_word_embeddings=False, max_position_embeddings=512), 256, (1, 140, 300)),
}


def draw_config(seed) -> tuple:
    if seed in CORNERS:
        sizes, page, lengths = CORNERS[seed]
        return _qwen3(**sizes), page, lengths
    rng = np.random.default_rng(1000 + seed)
    head_dim = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 192, 256, 512]))
    kv_heads = int(rng.integers(1, 5))
    group = int(rng.integers(1, 6))
    hidden = int(rng.integers(8, 40)) * int(rng.choice([2, 4, 8, 8]))
    config = _qwen3(
        num_hidden_layers=int(rng.integers(1, 4)), hidden_size=hidden, num_attention_heads=kv_heads * group,
        num_key_value_heads=kv_heads, head_dim=head_dim, intermediate_size=2 * int(rng.integers(10, 90)),
        vocab_size=int(rng.integers(90, 700)), rope_theta=float(10 ** rng.uniform(3, 7)),
        rms_norm_eps=float(10 ** rng.uniform(-7, -4)), tie_word_embeddings=bool(rng.integers(0, 2)),
        max_position_embeddings=512,
    )
    page = int(rng.choice([16, 32, 64, 128, 256]))
    lengths = (int(rng.integers(1, 40)), int(rng.integers(60, 200)), int(rng.integers(200, 330)))
    return config, page, lengths


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [*range(10), *CORNERS])
def test_a_random_configuration_matches_the_plain_model(tmp_path, seed, dtype):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.engine import Runner

    config, page, lengths = draw_config(seed)
    number = seed if isinstance(seed, int) else 77
    folder = make_model_folder(tmp_path, f"random{seed}", dtype=dtype, config=config, seed=number, norm_jitter=0.2,
                               std=0.05)
    cfg, weights = read_folder(folder)
    reqs = {f"r{i}": random_tokens(cfg["vocab_size"], n, 300 + 10 * number + i) for i, n in enumerate(lengths)}
    want = {rid: plain.forward(weights, cfg, toks) for rid, toks in reqs.items()}
    what = {k: cfg[k] for k in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim",
                                "intermediate_size", "vocab_size", "num_hidden_layers")}
    for cut, steps in (("whole", traces.whole(reqs)), ("tail", traces.tail_one_by_one(reqs, tail=6)),
                       ("mixed", traces.mixed(reqs, seed=number, tail=5, max_portion=70))):
        pages = -(-traces.peak_tokens(steps, page) // page)
        runner = Runner.from_folder(folder, dtype=dtype, page_size=page, num_pages=pages, max_requests=4)
        got, _ = traces.replay(runner, steps, cfg["vocab_size"])
        for rid, ref in want.items():
            ok, row, frac = rows_within(got[rid], ref, BOUND[dtype])
            assert ok, f"{what} page {page} {dtype}/{cut}: {rid} position {row} off by {frac:.3e} of its largest logit"
