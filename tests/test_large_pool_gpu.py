"""Cache tensors of more than 4 GiB, with the tested requests in the highest page ids: an
address computed in 32 bits anywhere between the block table and a key would show.  The
reference's pool has the same layout, ``[pages, page_size, kv_heads, head_dim]`` per layer
(/root/reference/src/pylon/kv/pool.py:36-44), and on this card the size that
/root/reference/src/pylon/engine.py:173-178 gives it is of this order."""
import numpy as np
import pytest
import torch

from tests import traces
from tests.helpers import _qwen3, make_model_folder, random_tokens, read_folder, rows_within
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu

# One layer of the published models' cache geometry: 8 key/value heads of 128, pages of 256.
WIDE = _qwen3(
    num_hidden_layers=1, hidden_size=96, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
    intermediate_size=160, vocab_size=283, rope_theta=1000000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, max_position_embeddings=2048,
)
PAGE = 256
LENGTHS = (300, 70, 1100, 513, 259)
BOUND = {"float32": 2e-5, "bfloat16": 2e-2}


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_requests_in_the_last_pages_of_a_pool_beyond_4_gib(tmp_path, dtype):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.engine import Runner

    folder = make_model_folder(tmp_path, "wide", dtype=dtype, config=WIDE, seed=3, norm_jitter=0.2, std=0.08)
    cfg, weights = read_folder(folder)
    reqs = {f"r{i}": random_tokens(cfg["vocab_size"], n, 70 + i) for i, n in enumerate(LENGTHS)}
    want = {rid: plain.forward(weights, cfg, toks) for rid, toks in reqs.items()}
    element = 2 if dtype == "bfloat16" else 4
    page_bytes = PAGE * 8 * 128 * element
    num_pages = (4 << 30) // page_bytes + 40  # each of K and V: 4 GiB and 40 pages
    assert num_pages * PAGE < 2 ** 31
    cuttings = {
        "whole": traces.whole(reqs),
        "tail32": traces.tail_one_by_one(reqs),
        "mixed": traces.mixed(reqs, seed=13, max_portion=300),
    }
    runner = Runner.from_folder(folder, dtype=dtype, page_size=PAGE, num_pages=num_pages, max_requests=8)
    group = runner.manager.groups[0]
    assert group.k[0].numel() * group.k[0].element_size() > 4 << 30
    spare = max(-(-traces.peak_tokens(steps, PAGE) // PAGE) for steps in cuttings.values())
    # A request that never runs takes the low page ids: the tested ones get the top of the pool.
    parked = runner.open("parked")
    parked.pages[0] = group.pool.acquire(num_pages - spare)
    assert max(parked.pages[0]) == num_pages - spare - 1
    assert (num_pages - spare) * page_bytes >= 1 << 32  # every tested page lies beyond 4 GiB
    for cut, steps in cuttings.items():
        got, reused = traces.replay(runner, steps, cfg["vocab_size"], idle=1)
        assert cut != "mixed" or reused, "the mixed trace was meant to use pages again"
        for rid, ref in want.items():
            ok, row, frac = rows_within(got[rid], ref, BOUND[dtype])
            assert ok, f"{dtype}/{cut}: request {rid} position {row} is off by {frac:.3e} of its largest logit"
    assert group.pool.free_pages == spare
    runner.close(parked)
    runner.manager.check()
