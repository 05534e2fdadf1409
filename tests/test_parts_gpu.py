"""Each part of a layer alone against its plain formula, and a model whose layers differ
(windows, a layer run twice, a run that borrows another run's cache)."""
import dataclasses

import numpy as np
import pytest
import torch

from tests.helpers import make_model_folder, random_tokens, read_folder
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")


def f64(t):
    return t.detach().cpu().to(torch.float64).numpy()


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def test_norm_part():
    from pylon_amd.config.specs import NormSpec
    from pylon_amd.parts import build_part

    norm = build_part("norm", NormSpec("rmsnorm", 72, 1e-5), dtype=torch.float32, device=DEV)
    w = 1 + 0.3 * rnd((72,), 1)
    norm.params["weight"].copy_(w)
    x, d = rnd((5, 72), 2), rnd((5, 72), 3)
    resid = x.clone().to(DEV)
    y = norm.add_forward(resid, d.to(DEV))
    assert np.allclose(f64(resid), f64(x) + f64(d), atol=1e-6)
    assert np.allclose(f64(y), plain.rms_norm(f64(x) + f64(d), f64(w), 1e-5), atol=1e-5)
    assert np.allclose(f64(norm.forward(x.to(DEV))), plain.rms_norm(f64(x), f64(w), 1e-5), atol=1e-5)


def test_feed_forward_part():
    from pylon_amd.config.specs import GatedFeedForwardSpec
    from pylon_amd.parts import build_part

    ff = build_part("feed_forward", GatedFeedForwardSpec(hidden_size=40, intermediate_size=56),
                    dtype=torch.float32, device=DEV)
    gate, up, down = rnd((56, 40), 4, 0.2), rnd((56, 40), 5, 0.2), rnd((40, 56), 6, 0.2)
    ff.params["gate_up"].copy_(torch.cat([gate, up]))
    ff.params["down"].copy_(down)
    x = rnd((7, 40), 7)
    got = ff.forward(x.to(DEV), None)
    want = plain.gated_feed_forward(f64(x), f64(gate), f64(up), f64(down))
    assert np.allclose(f64(got), want, atol=1e-5)
    with pytest.raises(ValueError, match="not supported"):
        build_part("feed_forward", GatedFeedForwardSpec(8, 8, activation="gelu"), dtype=torch.float32, device=DEV)


def test_feed_forward_part_whose_gate_up_rows_lie_apart_in_memory():
    """A bfloat16 model's fused gate/up matrix keeps 64 unused elements behind every row (its rows
    then do not meet in the same few memory channels: here a width whose rows are 8 KB), the parameter
    is the view without them, a load fills it like any other, and every product kernel that
    takes part at some row count reads it through its row stride."""
    from pylon_amd.config.specs import GatedFeedForwardSpec
    from pylon_amd.engine.runner import weight_bytes
    from pylon_amd.parts import build_part

    hidden, inter = 4096, 4608
    ff = build_part("feed_forward", GatedFeedForwardSpec(hidden_size=hidden, intermediate_size=inter),
                    dtype=torch.bfloat16, device=DEV)
    gate_up = ff.params["gate_up"]
    assert gate_up.shape == (2 * inter, hidden) and gate_up.stride() == (hidden + 64, 1)
    assert ff.params["down"].is_contiguous()
    exact = build_part("feed_forward", GatedFeedForwardSpec(hidden_size=hidden, intermediate_size=8),
                       dtype=torch.float32, device=DEV)
    assert exact.params["gate_up"].is_contiguous()  # the 32-bit path's rows are left as they are
    gate, up = rnd((inter, hidden), 4, 0.02).to(torch.bfloat16), rnd((inter, hidden), 5, 0.02).to(torch.bfloat16)
    down = rnd((hidden, inter), 6, 0.02).to(torch.bfloat16)
    gate_up[:inter].copy_(gate)   # as the loader does: a row range of the view
    gate_up[inter:].copy_(up)
    ff.params["down"].copy_(down)
    for rows in (3, 16, 40, 64, 100, 300):  # skinny or rows kernel, rows kernel, library
        x = rnd((rows, hidden), 7 + rows).to(torch.bfloat16)
        got = ff.forward(x.to(DEV), None)
        got = got.sum(0) if got.dim() == 3 else got
        want = plain.gated_feed_forward(f64(x), f64(gate), f64(up), f64(down))
        assert np.abs(f64(got) - want).max() <= 2e-2 * np.abs(want).max(), rows


def test_position_part_and_registry():
    from pylon_amd.config.specs import PositionSpec
    from pylon_amd.parts import build_part

    rope = build_part("position", PositionSpec("rope", theta=1e6, rotary_dim=32, max_positions=64),
                      dtype=torch.float32, device=DEV)
    inv, dim = rope.rotary()
    want = 1.0 / (np.float32(1e6) ** (np.arange(0, 32, 2, dtype=np.float32) / np.float32(32)))
    assert dim == 32 and np.allclose(inv.cpu().numpy(), want, rtol=1e-6)
    assert build_part("position", PositionSpec("none"), dtype=torch.float32, device=DEV).rotary() is None
    with pytest.raises(ValueError, match="no position of kind 'alibi'"):
        build_part("position", PositionSpec("alibi"), dtype=torch.float32, device=DEV)


def _attention_alone(window, qk_norm, rot):
    """The attention part over a cache it fills itself, against the plain formulas."""
    from pylon_amd.cache import CacheManager
    from pylon_amd.config.specs import AttentionSpec, PositionSpec
    from pylon_amd.engine.batch import MetadataArena, StepEntry, build_step
    from pylon_amd.parts import build_part

    hidden, nh, nkv, hd, tokens = 40, 6, 3, 16, 45
    position = PositionSpec("rope", theta=500.0, rotary_dim=rot, max_positions=512) if rot else PositionSpec("none")
    spec = AttentionSpec(hidden_size=hidden, n_heads=nh, n_kv_heads=nkv, head_dim=hd, scale=0.31,
                         position=position, qk_norm=qk_norm, qk_norm_eps=1e-4, window=window)
    att = build_part("mixer", spec, dtype=torch.float32, device=DEV)
    wq, wk, wv = rnd((nh * hd, hidden), 8, 0.3), rnd((nkv * hd, hidden), 9, 0.3), rnd((nkv * hd, hidden), 10, 0.3)
    wo = rnd((hidden, nh * hd), 11, 0.3)
    att.params["qkv"].copy_(torch.cat([wq, wk, wv]))
    att.params["out"].copy_(wo)
    qn, kn = 1 + 0.2 * rnd((hd,), 12), 1 + 0.2 * rnd((hd,), 13)
    if qk_norm:
        att.params["q_norm"].copy_(qn)
        att.params["k_norm"].copy_(kn)
    manager = CacheManager([att.cache_requirement()], page_size=16, num_pages=4, max_requests=2,
                           dtype=torch.float32, device=DEV)
    arena = MetadataArena(DEV)
    seq = manager.open("x")
    h = rnd((tokens, hidden), 14)
    outs = []
    for lo, hi in ((0, 20), (20, 21), (21, 45)):  # a portion, one token, a portion
        ctx = build_step([StepEntry(seq, [1] * (hi - lo), [])], manager, arena, vocab_size=10)
        outs.append(att.forward(h[lo:hi].contiguous().to(DEV), ctx, ctx.cache(0), True))
        manager.commit([(seq, hi - lo)])
    got = f64(torch.cat(outs))
    # the plain formulas
    x = f64(h)
    q = (x @ f64(wq).T).reshape(tokens, nh, hd).transpose(1, 0, 2)
    k = (x @ f64(wk).T).reshape(tokens, nkv, hd).transpose(1, 0, 2)
    v = (x @ f64(wv).T).reshape(tokens, nkv, hd).transpose(1, 0, 2)
    if qk_norm:
        q, k = plain.rms_norm(q, f64(qn), 1e-4), plain.rms_norm(k, f64(kn), 1e-4)
    if rot:
        cos, sin = plain.rope_tables(range(tokens), rot, 500.0)
        pad = np.ones((tokens, hd - rot)), np.zeros((tokens, hd - rot))
        # partial rotation: the first `rot` elements turn, the rest pass
        def turn(t):
            head, tail = t[..., :rot], t[..., rot:]
            return np.concatenate([plain.apply_rope(head, cos, sin), tail], axis=-1)
        q, k = turn(q), turn(k)
    ctxv = plain.causal_attention(q, k, v, 0.31, window)
    want = ctxv.transpose(1, 0, 2).reshape(tokens, nh * hd) @ f64(wo).T
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("window,qk_norm,rot", [(None, True, 16), (7, True, 16), (None, False, 0),
                                                (19, False, 8), (1, True, 16)])
def test_attention_part(window, qk_norm, rot):
    _attention_alone(window, qk_norm, rot)


def test_layers_that_differ_and_a_schedule_with_repeats_and_borrowing(tmp_path):
    """One model whose layers have different windows, with a layer run twice and a run
    that reads an earlier run's cache; cut into portions, against the plain model."""
    from pylon_amd.config import load_model_config
    from pylon_amd.config.specs import ScheduleEntry
    from pylon_amd.engine import Model, Runner, StepEntry
    from pylon_amd.weights import load_weights

    folder = make_model_folder(tmp_path, "B", dtype="float32", std=0.08)
    cfg, weights = read_folder(folder)
    arch, config = load_model_config(folder)
    spec = arch.model_spec(config)
    layers = list(spec.layers)
    layers[1] = dataclasses.replace(layers[1], mixer=dataclasses.replace(layers[1].mixer, window=9))
    schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2), ScheduleEntry(0), ScheduleEntry(2, cache=2),
                ScheduleEntry(1))
    spec = dataclasses.replace(spec, layers=tuple(layers), schedule=schedule)
    model = Model(spec, dtype=torch.float32, device=DEV)
    load_weights(model, arch, config, folder)
    runner = Runner(model, page_size=16, num_pages=9, max_requests=2)
    assert len(runner.manager.groups) == 2  # full attention and the windowed layer
    assert sorted(map(sorted, (g.cache_ids for g in runner.manager.groups))) == [[0, 2, 3], [1, 5]]
    toks = random_tokens(cfg["vocab_size"], 140, 9)
    want = plain.forward(weights, cfg, toks, schedule=[(0, None), (1, None), (2, None), (0, None), (2, 2), (1, None)],
                         windows={1: 9})
    seq = runner.open("s")
    outs, pos = [], 0
    for size in (33, 1, 1, 50, 2, 40, 13):
        outs.append(runner.step([StepEntry(seq, toks[pos:pos + size], list(range(size)))]).cpu().numpy())
        pos += size
        runner.manager.check()
    got = np.concatenate(outs)
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    # the windowed group holds far fewer pages than the full one
    assert len([p for p in seq.pages[1] if p >= 0]) <= 2 and len(seq.pages[0]) == 9
