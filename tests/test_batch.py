"""The tiles a step's tokens are cut into for the prompt-attention kernel."""
import numpy as np
import torch

from pylon_amd.cache import CacheManager
from pylon_amd.engine.batch import MetadataArena, StepEntry, build_step
from pylon_amd.parts.base import KVRequirement


def _step(counts, cached):
    manager = CacheManager([KVRequirement(n_kv_heads=1, head_dim=16)], page_size=4, num_pages=400,
                           max_requests=8, dtype=torch.float32, device="cpu")
    entries = []
    for i, (count, before) in enumerate(zip(counts, cached)):
        seq = manager.open(f"r{i}")
        if before:
            manager.reserve([(seq, before)])
            manager.commit([(seq, before)])
        entries.append(StepEntry(seq, [1] * count, []))
    return build_step(entries, manager, MetadataArena("cpu", capacity=1024), vocab_size=10)


def _check_cover(tiles, counts, cached, per_tile, skip):
    starts = np.concatenate([[0], np.cumsum(counts)])
    seen = np.zeros(starts[-1], dtype=int)
    for first, count, row, pos in tiles.tolist():
        assert 1 <= count <= per_tile and row >= skip
        assert starts[row] <= first and first + count <= starts[row + 1]  # one request only
        assert pos == cached[row] + first - starts[row]
        seen[first: first + count] += 1
    assert (seen[starts[skip]:] == 1).all() and (seen[: starts[skip]] == 0).all()


def test_tiles_cover_every_token_once_longest_context_first():
    counts, cached = [1, 1, 37, 5, 64, 130], [9, 0, 0, 31, 16, 3]
    ctx = _step(counts, cached)
    assert ctx.leading_singles == 2
    for per_tile in (4, 16, 32):
        for skip in (0, 2):
            tiles = ctx.token_tiles(per_tile, skip_rows=skip)
            _check_cover(tiles, counts, cached, per_tile, skip)
            ends = (tiles[:, 3] + tiles[:, 1]).tolist()
            assert ends == sorted(ends, reverse=True)


def test_folded_tiles_turn_every_second_run_round():
    counts, cached = [1, 1, 37, 5, 64, 130], [9, 0, 0, 31, 16, 3]
    ctx = _step(counts, cached)
    plain = (lambda t: (t[:, 3] + t[:, 1]).tolist())(ctx.token_tiles(4, skip_rows=2))
    for fold in (1, 3, 5, 1000):
        tiles = ctx.token_tiles(4, skip_rows=2, fold=fold)
        _check_cover(tiles, counts, cached, 4, 2)
        ends = (tiles[:, 3] + tiles[:, 1]).tolist()
        want = []
        for start in range(0, len(plain), fold):
            run = plain[start: start + fold]
            want += run[::-1] if (start // fold) % 2 else run
        assert ends == want
    assert ctx.token_tiles(4, skip_rows=2, fold=1000).tolist() == ctx.token_tiles(4, skip_rows=2).tolist()
