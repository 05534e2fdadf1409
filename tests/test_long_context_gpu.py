"""Contexts of the length the published configurations allow (262,144 positions): the attention
kernels over a quarter of a million cached keys with a few far keys made to stand out, the
rotation at positions beyond 2^16 and 2^20, and a request of eight thousand tokens through
the engine against the plain model."""

import numpy as np
import pytest
import torch

from tests import traces
from tests.helpers import _qwen3, make_model_folder, random_tokens, read_folder, rows_within
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.kernels import check_device, ops as _ops

    check_device()
    return _ops


def _long_cache(lengths, nkv, hd, page, seed):
    """Pages in scrambled order for requests of the given lengths; keys small and random,
    so that the few keys a test plants decide the result."""
    gen = torch.Generator(device=DEV).manual_seed(seed)
    per = [-(-n // page) for n in lengths]
    n_pages = sum(per) + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).to(torch.int32)
    table = torch.zeros((len(lengths), max(per)), dtype=torch.int32)
    cursor = 0
    for r, count in enumerate(per):
        table[r, :count] = perm[cursor: cursor + count]
        cursor += count
    kc = (torch.randn((n_pages, page, nkv, hd), generator=gen, device=DEV) * 0.05).to(torch.bfloat16)
    vc = torch.randn((n_pages, page, nkv, hd), generator=gen, device=DEV).to(torch.bfloat16)
    return kc, vc, table


def _reference(q, kc, vc, table_row, n, scale, window=None):
    """float64 attention of queries [heads, d] at position n-1 over the request's n keys."""
    page = kc.shape[1]
    pages = table_row[: -(-n // page)].to(DEV).long()
    keys = kc[pages].reshape(-1, kc.shape[2], kc.shape[3])[:n].double()  # [n, kv, d]
    vals = vc[pages].reshape(-1, vc.shape[2], vc.shape[3])[:n].double()
    lo = max(0, n - window) if window else 0
    group = q.shape[0] // keys.shape[1]
    out = torch.empty(q.shape, dtype=torch.float64, device=DEV)
    for h in range(q.shape[0]):
        s = keys[lo:, h // group] @ q[h].double() * scale
        out[h] = torch.softmax(s, 0) @ vals[lo:, h // group]
    return out


def _plant(kc, table, row, position, kv_head, vector):
    page = kc.shape[1]
    kc[int(table[row, position // page]), position % page, kv_head] = vector.to(kc.dtype)


@pytest.mark.parametrize("window", [None, 100_000])
def test_decode_attention_over_a_quarter_of_a_million_keys(ops, window):
    nh, nkv, hd, page = 4, 2, 128, 256
    lengths = [262_144 - 5, 131_073, 70_001]
    kc, vc, table = _long_cache(lengths, nkv, hd, page, seed=5)
    q = (torch.randn((len(lengths), nh, hd), generator=torch.Generator().manual_seed(6)) * 0.3).to(torch.bfloat16).to(DEV)
    # keys that match a query head strongly, spread over the whole length: the first page, the
    # places where 16-bit and 17-bit counts wrap, the last key
    for r, n in enumerate(lengths):
        for i, place in enumerate((3, 65_535, 65_536, n // 2 + 1, n - 40_000, n - 1)):
            if 0 <= place < n:
                head = i % nh
                _plant(kc, table, r, place, head // (nh // nkv), q[r, head].float() * (1.6 + 0.1 * i))
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32, device=DEV)
    scale = 1.0
    want = torch.stack([_reference(q[r], kc, vc, table[r], n, scale, window) for r, n in enumerate(lengths)])
    assert float(want.abs().max()) > 0.3  # the planted keys, not an average of noise, make the result
    chosen = ops.decode_launch(len(lengths), nkv, max(lengths) if window is None else window)
    for cuts, splits in {chosen, (1, 8), (64, 4), (7, 2)}:
        got = ops.attention_decode(q, kc, vc, table.to(DEV), None, positions, page_size=page, window=window,
                                   scale=scale, n_splits=splits, n_cuts=cuts)
        err = float((got.double() - want).abs().max())
        assert err <= 6e-3 * max(1.0, float(want.abs().max())), (cuts, splits, err)
    rows = torch.arange(len(lengths), dtype=torch.int32, device=DEV)
    general = ops.paged_attention(q, kc, vc, table.to(DEV), rows, positions, page_size=page, window=window, scale=scale)
    assert float((general.double() - want).abs().max()) <= 6e-3 * max(1.0, float(want.abs().max()))


def test_prompt_attention_of_a_portion_behind_a_quarter_of_a_million_keys(ops):
    nh, nkv, hd, page = 4, 2, 128, 256
    before, count = 262_144 - 200, 150
    kc, vc, table = _long_cache([before + count], nkv, hd, page, seed=8)
    q = (torch.randn((count, nh, hd), generator=torch.Generator().manual_seed(9)) * 0.3).to(torch.bfloat16).to(DEV)
    for i, (token, place) in enumerate(((0, 5), (0, 65_536), (70, 131_072), (149, before + 149), (149, before - 1),
                                        (33, before + 33), (100, 200_000))):
        head = i % nh
        _plant(kc, table, 0, place, head // (nh // nkv), q[token, head].float() * 1.8)
    per_tile = 128 // (nh // nkv)
    tiles = [(lo, min(per_tile, count - lo), 0, before + lo) for lo in range(0, count, per_tile)]
    got = ops.attention_prefill(q, kc, vc, table.to(DEV), torch.tensor(tiles, dtype=torch.int32, device=DEV),
                                page_size=page, window=None, scale=1.0, rows=128)
    for token in (0, 33, 70, 100, 149):
        want = _reference(q[token], kc, vc, table[0], before + token + 1, 1.0)
        err = float((got[token].double() - want).abs().max())
        assert err <= 1.2e-2 * max(1.0, float(want.abs().max())), (token, err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotation_at_positions_beyond_two_to_the_twentieth(ops, dtype):
    """The angle is the float32 product of position and inverse frequency, as the tables of
    /root/reference/src/pylon/model/layers.py:43-51 hold it; its sine and cosine must be those
    of that float32 number, also where it is hundreds of thousands of radians."""
    nh, nkv, hd = 3, 1, 64
    positions = [0, 65_535, 65_536, 131_071, 262_143, 1_048_577, 16_777_215]
    tokens = len(positions)
    g = torch.Generator().manual_seed(3)
    qkv = torch.randn((tokens, nh * hd), generator=g).to(dtype)  # queries only: nothing is stored
    inv_freq = 1.0 / (1_000_000.0 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))
    q = torch.empty((tokens, nh, hd), dtype=dtype, device=DEV)
    ops.qkv_prepare(qkv.to(DEV), q, None, None, n_heads=nh, n_kv_heads=nkv, head_dim=hd, q_weight=None,
                    k_weight=None, eps=1e-6, inv_freq=inv_freq.to(DEV), rot_dim=hd,
                    positions=torch.tensor(positions, dtype=torch.int32, device=DEV), slot_map=None, store_kv=False)
    raw = qkv.double().numpy().reshape(tokens, nh, hd)
    for t, pos in enumerate(positions):
        angle = (np.float32(pos) * inv_freq.numpy()).astype(np.float64)
        a, b = raw[t, :, : hd // 2], raw[t, :, hd // 2:]
        want = np.concatenate([a * np.cos(angle) - b * np.sin(angle), b * np.cos(angle) + a * np.sin(angle)], -1)
        err = np.abs(q[t].double().cpu().numpy() - want).max()
        assert err <= (2e-6 if dtype == torch.float32 else 6e-3) * np.abs(want).max(), (pos, err)


# Over eight thousand tokens the plain model is slow: few heads, two layers, a small vocabulary.
LONG = _qwen3(num_hidden_layers=2, hidden_size=64, num_attention_heads=2, num_key_value_heads=1, head_dim=128,
              intermediate_size=96, vocab_size=211, rope_theta=1_000_000.0, rms_norm_eps=1e-6,
              tie_word_embeddings=True, max_position_embeddings=16_384)


LENGTH = 8_501
PLACES = sorted({0, 1, 63, 64, 2047, 2048, 4095, 4096, 6143, 6144, 8191, 8192, *range(LENGTH - 12, LENGTH)})


@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    """One folder stored in bfloat16 (a float32 model widens it exactly), the long and the short
    request, and the plain model's logits at the compared places: the plain model takes most
    of a minute over eight thousand tokens, so both precisions share it."""
    folder = make_model_folder(tmp_path_factory.mktemp("long"), "long", dtype="bfloat16", config=LONG, seed=71,
                               norm_jitter=0.2, std=0.06)
    cfg, weights = read_folder(folder)
    tokens = random_tokens(cfg["vocab_size"], LENGTH, 72)
    short = random_tokens(cfg["vocab_size"], 90, 73)
    return folder, cfg, tokens, short, plain.forward(weights, cfg, tokens)[PLACES], plain.forward(weights, cfg, short)


@pytest.mark.parametrize("dtype,bound", [("float32", 2e-5), ("bfloat16", 2e-2)])
def test_a_request_of_eight_thousand_tokens_matches_the_plain_model(long_model, dtype, bound):
    """Fed in portions of 2,048 with the last tokens one by one, beside a short request that
    comes and goes so that pages are used again; compared at places spread over its length."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.engine import Runner

    folder, cfg, tokens, short, ref, ref_short = long_model
    length, page, places = LENGTH, 64, PLACES
    steps, pos = [], 0
    while pos < length - 8:
        size = min(2048, length - 8 - pos)
        want = [p - pos for p in places if pos <= p < pos + size]
        entries = [{"id": "long", "tokens": tokens[pos: pos + size], "want": want}]
        turn = len(steps) % 3
        if turn == 0:
            entries.append({"id": f"s{len(steps)}", "tokens": short[:50], "want": list(range(50))})
        elif turn == 1:
            entries.insert(0, {"id": f"s{len(steps) - 1}", "tokens": short[50:], "want": list(range(40))})
        steps.append({"step": len(steps), "entries": entries, "end": [f"s{len(steps) - 1}"] if turn == 1 else []})
        pos += size
    for p in range(pos, length):
        steps.append({"step": len(steps), "entries": [{"id": "long", "tokens": [tokens[p]], "want": [0]}],
                      "end": ["long"] if p == length - 1 else []})
    pages = -(-length // page) + 3  # the short request's two pages pass from hand to hand
    runner = Runner.from_folder(folder, dtype=dtype, page_size=page, num_pages=pages, max_requests=3)
    got, _ = traces.replay(runner, steps, cfg["vocab_size"])
    ok, row, frac = rows_within(got["long"], ref, bound)
    assert ok, f"{dtype}: position {places[row]} off by {frac:.3e} of its largest logit"
    for rid, rows in got.items():
        if rid != "long":
            ok, row, frac = rows_within(rows, ref_short, bound)
            assert ok, f"{dtype}: {rid} position {row} off by {frac:.3e}"
