"""The cache manager on the CPU: pages, block tables, windows, state slots, and the
step's metadata vectors."""
import random

import pytest
import torch

from pylon_amd.cache import CacheManager, OutOfPages, OutOfSlots, PagePool, StateSlots
from pylon_amd.cache.manager import FREED
from pylon_amd.engine.batch import MetadataArena, StepEntry, build_step
from pylon_amd.parts.base import KVRequirement, StateRequirement

FULL = KVRequirement(n_kv_heads=1, head_dim=16)


def make(requirements=(FULL, FULL), page_size=4, num_pages=8, max_requests=4):
    return CacheManager(list(requirements), page_size=page_size, num_pages=num_pages,
                        max_requests=max_requests, dtype=torch.float32, device="cpu")


def feed(manager, seq, count):
    manager.reserve([(seq, count)])
    manager.commit([(seq, count)])


def test_pool_hands_out_in_order_and_reuses_the_last_released_first():
    # /root/reference/tests/test_paged_attention.py:70-89
    pool = PagePool(4)
    assert pool.acquire(2) == [0, 1]
    pool.release(0)
    assert pool.acquire(1) == [0]
    assert pool.acquire(2) == [2, 3]
    with pytest.raises(OutOfPages):
        pool.acquire(1)
    pool.check()


def test_pool_refuses_double_release_and_foreign_pages():
    pool = PagePool(3)
    (page,) = pool.acquire(1)
    pool.retain(page)
    pool.release(page)
    assert pool.free_pages == 2  # still held once
    pool.release(page)
    assert pool.free_pages == 3
    with pytest.raises(RuntimeError, match="more often"):
        pool.release(page)
    with pytest.raises(ValueError):
        pool.release(7)
    with pytest.raises(RuntimeError, match="free and cannot be retained"):
        pool.retain(page)
    with pytest.raises(ValueError):
        PagePool(0)


def test_the_token_after_a_full_page_takes_the_next_page():
    # /root/reference/tests/test_paged_attention.py:53-68 (there with 256-token pages)
    m = make(page_size=4)
    seq = m.open("r")
    feed(m, seq, 4)
    assert seq.pages == [[0]] and seq.length == 4
    feed(m, seq, 1)
    assert seq.pages == [[0, 1]] and seq.length == 5
    m.close(seq)
    assert m.free_pages == 8
    other = m.open("s")
    feed(m, other, 1)
    assert other.pages == [[1]]  # the page released last comes out first
    m.check()


def test_reserve_checks_every_entry_before_taking_a_page():
    m = make(num_pages=3)
    a, b = m.open("a"), m.open("b")
    feed(m, a, 4)
    with pytest.raises(OutOfPages):
        m.reserve([(a, 4), (b, 8)])  # needs 1 + 2 pages, 2 are free
    assert a.pages == [[0]] and b.pages == [[]] and m.free_pages == 2 and a._pending is None
    with pytest.raises(ValueError, match="distinct"):
        m.reserve([(a, 1), (a, 1)])
    with pytest.raises(ValueError, match="at least one"):
        m.reserve([(a, 0)])
    m.reserve([(a, 1)])
    with pytest.raises(ValueError, match="pending"):
        m.reserve([(a, 1)])
    m.cancel([(a, 1)])
    assert a.pages == [[0]] and a.length == 4 and m.free_pages == 2
    capped = m.open("c", capacity=5)
    with pytest.raises(ValueError, match="capacity"):
        m.reserve([(capped, 6)])
    m.check()


def test_close_twice_and_reopen():
    m = make()
    seq = m.open("a")
    with pytest.raises(ValueError, match="already has a cache"):
        m.open("a")
    feed(m, seq, 9)
    m.close(seq)
    with pytest.raises(RuntimeError, match="closed twice"):
        m.close(seq)
    with pytest.raises(ValueError, match="has been closed"):
        m.reserve([(seq, 1)])
    m.open("a")
    m.check()


def test_groups_have_pages_of_their_own_and_a_window_gives_pages_back():
    window = KVRequirement(n_kv_heads=1, head_dim=16, window=6)
    wide = KVRequirement(n_kv_heads=2, head_dim=32)
    m = make(requirements=(FULL, window, FULL, wide, None), page_size=4, num_pages=6)
    assert [g.cache_ids for g in m.groups] == [[0, 2], [1], [3]]
    assert m.groups[2].k[3].shape == (6, 4, 2, 32) and m.groups[0].k[2].shape == (6, 4, 1, 16)
    assert m.view(4).k is None and m.view(1).group == 1
    seq = m.open("r")
    feed(m, seq, 9)  # positions 0..8; the next token (9) sees keys 4..9: page 0 is dead
    assert seq.pages[0] == [0, 1, 2] and seq.pages[2] == [0, 1, 2]
    assert seq.pages[1] == [FREED, 1, 2]
    assert m.groups[1].pool.free_pages == 4 and m.groups[0].pool.free_pages == 3
    feed(m, seq, 1)  # length 10: first needed key 5 -> page 1 (keys 4..7) still live
    assert seq.pages[1] == [FREED, 1, 2]
    feed(m, seq, 3)  # length 13: first needed key 8 -> page 1 dead; page 3 taken (the freed page 0)
    assert seq.pages[1] == [FREED, FREED, 2, 0]
    m.check()
    # a long request in a windowed group never holds more than ceil((window+chunk)/page)+1 pages
    for _ in range(40):
        feed(m, seq, 1) if m.groups[0].pool.free_pages else None
        if not m.groups[0].pool.free_pages:
            break
    live = [p for p in seq.pages[1] if p != FREED]
    assert len(live) <= 3
    m.close(seq)
    assert all(g.pool.free_pages == 6 for g in m.groups)
    m.check()


def test_random_orders_never_lose_or_double_a_page():
    rnd = random.Random(5)
    window = KVRequirement(n_kv_heads=1, head_dim=16, window=5)
    for trial in range(30):
        m = make(requirements=(FULL, window), page_size=4, num_pages=rnd.randint(3, 12), max_requests=5)
        live = {}
        for step in range(120):
            action = rnd.random()
            if action < 0.25 and len(live) < 5:
                rid = f"{trial}-{step}"
                live[rid] = m.open(rid)
            elif action < 0.4 and live:
                rid = rnd.choice(sorted(live))
                m.close(live.pop(rid))
            elif live:
                chosen = rnd.sample(sorted(live), rnd.randint(1, len(live)))
                entries = [(live[r], rnd.choice([1, 1, 2, 3, 7])) for r in chosen]
                before = [(list(map(list, s.pages)), s.length) for s, _ in entries]
                try:
                    m.reserve(entries)
                except OutOfPages:
                    assert before == [(list(map(list, s.pages)), s.length) for s, _ in entries]
                else:
                    if rnd.random() < 0.15:
                        m.cancel(entries)
                    else:
                        m.commit(entries)
            m.check()
        for seq in list(live.values()):
            m.close(seq)
        m.check()
        assert all(g.pool.free_pages == g.pool.num_pages for g in m.groups)
        assert m.slots.free_slots == 5


def test_state_slots():
    slots = StateSlots(2)
    t = slots.add_state(3, (4,), torch.float32, "cpu")
    a = slots.acquire()
    t[a] = 5.0
    b = slots.acquire()
    with pytest.raises(OutOfSlots):
        slots.acquire()
    slots.release(a)
    with pytest.raises(RuntimeError):
        slots.release(a)
    again = slots.acquire()
    assert again == a and float(t[again].abs().sum()) == 0.0  # cleared when handed out
    slots.check()
    m = make(requirements=(FULL, StateRequirement((3, 2), torch.float32)), max_requests=2)
    assert m.view(1).state.shape == (2, 3, 2) and m.view(1).k is None
    s1, s2 = m.open("a"), m.open("b")
    assert {s1.slot, s2.slot} == {0, 1}
    with pytest.raises(OutOfSlots):
        m.open("c")
    m.close(s1)
    assert m.open("c").slot == s1.slot


def _ctx(manager, entries, **kw):
    return build_step(entries, manager, MetadataArena("cpu", capacity=256), vocab_size=100, **kw)


def test_step_metadata_vectors_of_the_reference():
    # lengths (3, 7) plus one token each (/root/reference/tests/test_paged_attention.py:91-112)
    m = make(page_size=4, num_pages=8)
    a, b = m.open("a"), m.open("b")
    feed(m, a, 3)
    feed(m, b, 7)
    ctx = _ctx(m, [StepEntry(a, [5], [0]), StepEntry(b, [6], [0])])
    assert ctx.seq_lens.tolist() == [4, 8] and ctx.row_start.tolist() == [0, 1, 2]
    assert ctx.positions.tolist() == [3, 7] and ctx.tok_row.tolist() == [0, 1]
    assert ctx.seq_lens.dtype == torch.int32 and ctx.row_start.dtype == torch.int32
    assert ctx.logit_idx.tolist() == [0, 1] and ctx.decode_only
    assert ctx.cache(0).block_table.tolist() == [[0, 0], [1, 2]]
    assert ctx.cache(0).slot_map.tolist() == [0 * 4 + 3, 2 * 4 + 3]
    m.commit([(a, 1), (b, 1)])
    # lengths (0, page) -> positions [0, page], the second row's token opens its second page
    # (/root/reference/tests/test_cuda_graph_decode.py:79-100, there with 256-token pages)
    m2 = make(page_size=4, num_pages=8)
    c, d = m2.open("c"), m2.open("d")
    feed(m2, d, 4)
    ctx = _ctx(m2, [StepEntry(c, [1], [0]), StepEntry(d, [2], [0])])
    assert ctx.positions.tolist() == [0, 4] and ctx.seq_lens.tolist() == [1, 5]
    assert ctx.row_first.tolist() == [1, 0]
    assert ctx.cache(0).slot_map.tolist() == [c.pages[0][0] * 4 + 0, d.pages[0][1] * 4 + 0]


def test_mixed_step_metadata_and_refusals():
    m = make(page_size=4, num_pages=8)
    a, b = m.open("a"), m.open("b")
    feed(m, a, 6)
    ctx = _ctx(m, [StepEntry(a, [9], [0]), StepEntry(b, [1, 2, 3, 4, 5], [1, 4])])
    assert ctx.tokens == 6 and ctx.rows == 2 and not ctx.decode_only
    assert ctx.token_ids.tolist() == [9, 1, 2, 3, 4, 5]
    assert ctx.positions.tolist() == [6, 0, 1, 2, 3, 4]
    assert ctx.tok_row.tolist() == [0, 1, 1, 1, 1, 1]
    assert ctx.logit_idx.tolist() == [0, 2, 5] and ctx.n_logits == 3
    assert ctx.max_count == 5 and ctx.max_len == 7
    table = ctx.cache(1).block_table.tolist()
    assert table[0] == a.pages[0] and table[1] == b.pages[0]
    slots = ctx.cache(0).slot_map.tolist()
    assert slots[0] == a.pages[0][1] * 4 + 2 and slots[5] == b.pages[0][1] * 4 + 0
    m.commit([(a, 1), (b, 5)])
    free = m.free_pages
    for bad in ([StepEntry(a, [100], [0])], [StepEntry(a, [-1], [0])], [StepEntry(a, [1], [1])],
                [StepEntry(a, [], [])], []):
        with pytest.raises(ValueError):
            _ctx(m, bad)
        assert m.free_pages == free and a._pending is None
    with pytest.raises(OutOfPages):
        _ctx(m, [StepEntry(b, list(range(40)), [])])
    assert m.free_pages == free
    m.check()


def test_a_failure_after_the_pages_were_taken_gives_them_back():
    # the metadata upload fails (as a device error would): the step's pages return to the
    # pool, no append stays pending, and the next step runs
    m = make(page_size=4, num_pages=8)
    a = m.open("a")
    feed(m, a, 3)
    free = m.free_pages

    class FailingArena(MetadataArena):
        def upload(self, index, size, into=None):
            raise RuntimeError("device lost")

    with pytest.raises(RuntimeError, match="device lost"):
        build_step([StepEntry(a, [1, 2, 3], [2])], m, FailingArena("cpu", capacity=256), vocab_size=100)
    assert m.free_pages == free and a._pending is None
    m.check()
    with pytest.raises(ValueError, match="block table holds"):
        _ctx(m, [StepEntry(a, [1, 2, 3], [2])], width=1)
    assert m.free_pages == free and a._pending is None
    ctx = _ctx(m, [StepEntry(a, [1, 2, 3], [2])])
    assert ctx.positions.tolist() == [3, 4, 5]
    m.commit([(a, 3)])
    m.check()


def test_a_replay_that_raises_leaves_the_cache_as_it_was():
    from pylon_amd.engine.graphs import DecodeGraphs

    m = make(page_size=4, num_pages=8)
    a = m.open("a")
    feed(m, a, 4)  # the next token opens a second page
    free = m.free_pages

    class Spec:
        vocab_size = 100

    class FakeModel:
        spec = Spec()
        device = torch.device("cpu")

    class BrokenGraph:
        def replay(self):
            raise RuntimeError("replay failed")

    graphs = DecodeGraphs.__new__(DecodeGraphs)
    graphs.model, graphs.manager, graphs.arena = FakeModel(), m, MetadataArena("cpu", capacity=256)
    graphs.chosen, graphs.width, graphs.max_batch = None, 4, 4
    graphs.failed, graphs.replays, graphs.last_logit_slots = set(), 0, None
    block = torch.empty(256, dtype=torch.int32)
    graphs.captured = {graphs.key(1, 512): (BrokenGraph(), block, None, None)}
    with pytest.raises(RuntimeError, match="replay failed"):
        graphs.run([StepEntry(a, [7], [0])])
    assert m.free_pages == free and a._pending is None and a.length == 4
    m.check()
    ctx = _ctx(m, [StepEntry(a, [7], [0])])
    assert ctx.positions.tolist() == [4]


def test_a_budget_of_bytes_becomes_pages_per_group():
    """Every group holds the same requests, so every group gets the same number of pages,
    except that a group with a window never gets more than it can use; fixed-size state is
    taken off the budget first (by the caller)."""
    from types import SimpleNamespace as G

    from pylon_amd.cache.manager import plan_pool

    full, wide = G(bytes_per_token=100, window=None), G(bytes_per_token=300, window=None)
    kw = dict(page_size=4, max_requests=2, max_positions=None, chunk=8)
    # one group: the reference's budget // bytes of a page
    assert plan_pool(10_000, [full], **kw) == [10_000 // 400]
    # two groups that keep everything: one page of each costs 400 + 1200 bytes
    assert plan_pool(16_000, [full, wide], **kw) == [10, 10]
    assert plan_pool(15_999, [full, wide], **kw) == [9, 9]
    # a position limit caps them: two requests of 20 tokens are ten pages
    assert plan_pool(10 ** 9, [full, wide], page_size=4, max_requests=2, max_positions=20, chunk=8) == [10, 10]
    # a window of 6 with portions of 8: per request pages_for(14) + 1 = 5 pages, so ten; what it
    # does not need goes to the group beside it: 10 * 1200 + P * 400 <= 20,000 -> P = 20
    window = G(bytes_per_token=300, window=6)
    assert plan_pool(20_000, [full, window], **kw) == [20, 10]
    assert plan_pool(8_000, [full, window], **kw) == [5, 5]  # below the window's cap both get P
    with pytest.raises(RuntimeError, match="Not enough GPU memory"):
        plan_pool(1_599, [full, wide], **kw)
    assert plan_pool(123, [], **kw) == []
    # the manager takes one count per group, and admission counts with the largest
    m = CacheManager((FULL, KVRequirement(1, 16, window=6)), page_size=4, num_pages=[20, 10], max_requests=2,
                     dtype=torch.float32)
    assert [g.pool.num_pages for g in m.groups] == [20, 10] and m.num_pages == 20
    assert m.groups[1].k[1].shape[0] == 10
    with pytest.raises(ValueError, match="page counts"):
        CacheManager((FULL,), page_size=4, num_pages=[20, 10], max_requests=2, dtype=torch.float32)


def test_fixed_size_state_is_put_back_after_a_failed_step():
    m = make(requirements=(FULL, StateRequirement((3,), torch.float32)), max_requests=3)
    a, b, c = m.open("a"), m.open("b"), m.open("c")
    state = m.view(1).state
    state[a.slot], state[b.slot], state[c.slot] = 1.0, 2.0, 3.0
    saved = m.snapshot_state([c, a])
    state[a.slot] += 10.0  # what a mixer does before a later layer fails
    state[c.slot] += 10.0
    state[b.slot] += 10.0  # not part of the step: not put back
    m.restore_state(saved)
    assert state[a.slot].tolist() == [1.0] * 3 and state[c.slot].tolist() == [3.0] * 3
    assert state[b.slot].tolist() == [12.0] * 3
    # a model of keys and values only copies nothing
    plain_manager = make()
    assert plain_manager.snapshot_state([plain_manager.open("x")]) is None
    plain_manager.restore_state(None)
