"""The cache manager: no page lost, held twice or freed twice, under random orders of requests; windows; slots."""
import random

import numpy as np
import pytest
from hypothesis import given, settings
from hypothesis import strategies as st

from atoma_infer_amd.cache import CacheError, CacheManager, GroupGeometry, OutOfPages


def test_allocate_grow_free():
    """Mirrors backends/vllm/src/block_manager.rs:1162-1552 (allocate, append, free) for one group."""
    m = CacheManager([GroupGeometry(4, 6)], 2)
    assert m.add(10) == 0
    m.reserve(10, 9)                       # 3 pages
    assert m.table(10) == [0, 1, 2] and m.num_free_pages() == 3
    m.reserve(10, 9)                       # idempotent
    m.reserve(10, 12)                      # still 3 pages
    assert m.num_free_pages() == 3
    m.reserve(10, 13)                      # a 4th
    assert m.table(10) == [0, 1, 2, 3] and m.reserved_len(10) == 13
    m.check()
    assert m.can_reserve(10, 24) and not m.can_reserve(10, 25)
    with pytest.raises(OutOfPages):
        m.reserve(10, 25)
    assert m.table(10) == [0, 1, 2, 3]     # nothing taken by the failed call
    m.free(10)
    assert m.num_free_pages() == 6 and m.num_free_slots() == 2 and m.num_requests() == 0
    m.check()


def test_double_free_and_unknown_requests_are_errors():
    """backends/vllm/src/block_allocator.rs:147-229: freeing twice is an error."""
    m = CacheManager([GroupGeometry(4, 4)], 1)
    m.add(1)
    m.reserve(1, 5)
    m.free(1)
    with pytest.raises(CacheError):
        m.free(1)
    with pytest.raises(CacheError):
        m.reserve(2, 4)
    with pytest.raises(CacheError):
        m.table(2)
    m.add(3)
    with pytest.raises(CacheError):
        m.add(3)
    with pytest.raises(OutOfPages):
        m.add(4)                           # the only slot is taken
    m.check()


def test_freed_pages_are_used_again_last_freed_first():
    m = CacheManager([GroupGeometry(2, 4)], 4)
    m.add(1)
    m.reserve(1, 4)                        # pages 0, 1
    m.add(2)
    m.reserve(2, 2)                        # page 2
    m.free(1)
    m.add(3)
    m.reserve(3, 6)
    assert m.table(3) == [0, 1, 3]         # the freed pages first, in ascending order of position
    m.check()


def test_groups_reserve_together_or_not_at_all():
    m = CacheManager([GroupGeometry(4, 8), GroupGeometry(4, 2)], 2)
    m.add(1)
    with pytest.raises(OutOfPages):
        m.reserve(1, 12)                   # group 1 has only 2 pages
    assert m.num_free_pages(0) == 8 and m.num_free_pages(1) == 2
    m.reserve(1, 8)
    assert m.table(1, 0) == [0, 1] and m.table(1, 1) == [0, 1]
    assert m.fits_at_all(8) and not m.fits_at_all(9)


def test_window_gives_pages_back_while_running():
    m = CacheManager([GroupGeometry(4, 16, None), GroupGeometry(4, 4, 6)], 1)
    m.add(1)
    length = 0
    for step in range(40):
        length += 1
        m.reserve(1, length)
        m.release_behind(1, length)
        m.check()
        # a window of 6 tokens over pages of 4 never needs more than 3 live pages
        live = [p for p in m.table(1, 1) if p >= 0]
        assert len(live) <= 3
        first_needed = max(0, length - 6 + 1)
        assert all(p >= 0 for p in m.table(1, 1)[first_needed // 4:])
    assert len(m.table(1, 0)) == 10 and all(p >= 0 for p in m.table(1, 0))
    m.free(1)
    assert m.num_free_pages(1) == 4 and m.num_free_pages(0) == 16
    m.check()


def test_fill_step_slots_and_tables():
    m = CacheManager([GroupGeometry(4, 8)], 4)
    m.add(7)
    m.add(9)
    m.reserve(9, 3)
    m.reserve(7, 10)
    ids = np.array([7, 9], dtype=np.int64)
    starts, counts = np.array([6, 0], dtype=np.int32), np.array([4, 3], dtype=np.int32)
    sm = np.full(7, -9, dtype=np.int32)
    bt = np.full((2, 3), -9, dtype=np.int32)
    m.fill_step(0, ids, starts, counts, sm, bt)
    t7, t9 = m.table(7), m.table(9)
    assert bt.tolist() == [t7, t9 + [0, 0]]
    want = [t7[p // 4] * 4 + p % 4 for p in range(6, 10)] + [t9[0] * 4 + p for p in range(3)]
    assert sm.tolist() == want
    with pytest.raises(CacheError):
        m.fill_step(0, ids, np.array([9, 0], dtype=np.int32), counts, sm, bt)   # position 12 has no page


@settings(max_examples=60, deadline=None)
@given(seed=st.integers(0, 10_000), page=st.sampled_from([1, 4, 16]), pages=st.integers(4, 40),
       window=st.sampled_from([None, 3, 17]))
def test_random_orders_keep_the_books(seed, page, pages, window):
    rng = random.Random(seed)
    m = CacheManager([GroupGeometry(page, pages), GroupGeometry(page, pages, window)], 5)
    live = {}
    next_id = 0
    for _ in range(200):
        op = rng.random()
        if op < 0.25 and m.num_free_slots() > 0:
            m.add(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.75 and live:
            r = rng.choice(list(live))
            new = live[r] + rng.randint(1, 3 * page)
            if m.can_reserve(r, new):
                m.reserve(r, new)
                live[r] = new
                if rng.random() < 0.7:
                    m.release_behind(r, new)
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(r, new)
        elif live:
            r = rng.choice(list(live))
            m.free(r)
            del live[r]
        m.check()
        held = sum(-(-n // page) for n in live.values())
        assert m.num_free_pages(0) == pages - held
        assert m.num_free_pages(1) >= pages - held
        assert m.num_requests() == len(live) and m.num_free_slots() == 5 - len(live)
    for r in list(live):
        m.free(r)
    m.check()
    assert m.num_free_pages(0) == pages and m.num_free_pages(1) == pages and m.num_free_slots() == 5


def test_plan_cache_groups_layers_by_their_needs():
    from atoma_infer_amd.cache import plan_cache
    from atoma_infer_amd.config import LlamaConfig
    from atoma_infer_amd.models import LayerCall
    from atoma_infer_amd.models.llama import build_llama
    from util import TINY_B
    spec = build_llama(LlamaConfig.from_dict(TINY_B))
    plan = plan_cache(spec)
    assert len(plan.groups) == 1 and plan.groups[0].calls == [0, 1, 2]
    assert plan.bytes_per_token(2) == 2 * 3 * 3 * 32 * 2
    # a layer named twice has two entries; a call that reads another call's cache has none of its own
    spec.run_order = [LayerCall(0), LayerCall(1), LayerCall(1), LayerCall(2, kv_from=0)]
    spec.__post_init__()
    plan = plan_cache(spec)
    assert plan.groups[0].calls == [0, 1, 2]
    assert plan.where[3] == (0, 0, False) and plan.where[2] == (0, 2, True)
    # a window makes a group of its own
    spec.layers[2][1].mixer.window = 8
    spec.run_order = [LayerCall(0), LayerCall(1), LayerCall(2)]
    plan = plan_cache(spec)
    assert [g.spec.window for g in plan.groups] == [None, 8] and plan.where[2] == (1, 0, True)
    with pytest.raises(ValueError):
        spec.run_order = [LayerCall(0), LayerCall(2, kv_from=0)]   # needs differ
        spec.__post_init__()


@pytest.mark.parametrize("page,head", [(16, 64), (16, 48), (16, 16), (4, 16), (16, 256), (16, 80), (8, 32), (1, 32),
                                       (32, 64), (64, 128), (48, 80), (24, 32)])
def test_tile_layout_is_a_permutation_and_serves_the_mfma_lanes(page, head):
    import torch
    from atoma_infer_amd.cache.layout import (key_index, pack_keys, pack_values, unpack_keys, unpack_values,
                                               value_index)
    ki, vi = key_index(page, head), value_index(page, head)
    assert sorted(ki.reshape(-1).tolist()) == list(range(page * head))
    assert sorted(vi.reshape(-1).tolist()) == list(range(page * head))
    k, v = torch.randn(3, page, head), torch.randn(3, head, page)
    assert torch.equal(unpack_keys(pack_keys(k), page, head), k)
    assert torch.equal(unpack_values(pack_values(v), page, head), v)
    # a lane's 8 columns of a key are contiguous; with pages of 16, 32, 48, ... tokens a lane's 8 key slots of a value
    # column too, in every run of 16 tokens, and a run is laid out as a page of 16 tokens
    for t in range(page):
        for d0 in range(0, head, 8):
            assert ki[t, d0:d0 + 8].tolist() == list(range(int(ki[t, d0]), int(ki[t, d0]) + 8))
    if page % 16 == 0:
        v16 = value_index(16, head)
        for run in range(page // 16):
            assert torch.equal(vi[:, run * 16: run * 16 + 16], v16 + run * 16 * head)
            for d in range(head):
                for hg in (0, 1):
                    slots = [int(vi[d, run * 16 + hg * 4 + i]) for i in range(4)] + \
                            [int(vi[d, run * 16 + 8 + hg * 4 + i]) for i in range(4)]
                    assert slots == list(range(slots[0], slots[0] + 8)) and slots[0] % 8 == 0


def test_admission_with_a_window_counts_what_everyone_will_need():
    """Without a window, admission asks for the first portion's pages only.  With one, also for the window and a
    page of the newcomer and for what every request already held still lacks of its own."""
    m = CacheManager([GroupGeometry(4, 8)], 4)
    assert m.can_admit(100, 32) and not m.can_admit(100, 33)
    w = CacheManager([GroupGeometry(4, 8, window=10)], 4)           # a request in full swing needs 3 + 1 pages
    assert w.can_admit(100, 32) and not w.can_admit(100, 33)         # the first portion, all of it, at once
    w.add(1)
    w.reserve(1, 4)                                                  # holds 1 page, lacks 3 of its 4
    assert w.can_admit(100, 4)                                       # 4 (own) + 3 (lacking) <= 7 free
    w.add(2)
    w.reserve(2, 4)                                                  # 6 free; those there lack 3 each
    assert not w.can_admit(100, 4)                                   # 4 + 6 > 6
    assert not w.can_admit(4, 4)                                     # even a one-page request: 1 + 6 > 6
    w.reserve(1, 16)
    w.reserve(2, 12)                                                 # 1 free; they lack 0 and 1
    assert not w.can_admit(4, 4)
    w.free(2)
    assert w.can_admit(100, 4) and w.can_admit(100, 16) and not w.can_admit(100, 17)
    w.check()


@pytest.mark.parametrize("seed", range(8))
def test_a_step_packed_in_one_call_equals_the_arrays_made_one_by_one(seed):
    """``reserve_all`` / ``pack_step`` / ``release_behind_all`` against per-entry calls and arrays filled here."""
    rng = random.Random(seed)
    groups = [GroupGeometry(4, 200), GroupGeometry(16, 60, window=rng.choice([None, 24]))]
    one, two = CacheManager(groups, 8), CacheManager(groups, 8)
    held = {}
    for step in range(12):
        ids = [r for r in range(6) if rng.random() < 0.7]
        if not ids:
            continue
        rng.shuffle(ids)
        for r in ids:
            if r not in held:
                held[r] = 0
                assert one.add(r) == two.add(r)
        counts = [rng.choice([1, 1, 2, 7, 20]) for _ in ids]
        starts = [held[r] for r in ids]
        wants = [sorted(rng.sample(range(c), rng.randint(0, min(c, 3)))) for c in counts]
        feeds = [rng.randint(0, 9) if c == 1 and rng.random() < 0.3 else -1 for c in counts]
        tokens = [[rng.randrange(1000) for _ in range(c)] for c in counts]
        a_ids = np.asarray(ids, dtype=np.int64)
        a_starts, a_counts = np.asarray(starts, dtype=np.int32), np.asarray(counts, dtype=np.int32)
        for r, s0, c in zip(ids, starts, counts):
            one.reserve(r, s0 + c)
        two.reserve_all(a_ids, a_starts, a_counts)
        s, t, n_want = len(ids), sum(counts), sum(len(w) for w in wants)
        max_blocks = -(-max(s0 + c for s0, c in zip(starts, counts)) // 4)
        # the layout of the engine's staging buffer, with gaps of three between the arrays to catch overruns
        sizes = [t, t, t, s + 1, s, s, n_want, 2 * t, 2 * s * max_blocks, 2 * s]
        offs, total = [], 0
        for n in sizes:
            offs.append(total)
            total += n + 3
        buf = np.full(total, -7, dtype=np.int32)
        n_feed = two.pack_step(a_ids, a_starts, a_counts, np.asarray(sum(tokens, []), dtype=np.int32),
                               np.asarray(feeds, dtype=np.int32), np.asarray([len(w) for w in wants], dtype=np.int32),
                               np.asarray(sum(wants, []), dtype=np.int32), buf, np.asarray(offs, dtype=np.int64),
                               max_blocks)
        want = np.full(total, -7, dtype=np.int32)
        row, wi, pairs = 0, 0, []
        for e, (r, s0, c) in enumerate(zip(ids, starts, counts)):
            want[offs[0] + row: offs[0] + row + c] = tokens[e]
            want[offs[1] + row: offs[1] + row + c] = range(s0, s0 + c)
            want[offs[2] + row: offs[2] + row + c] = e
            want[offs[3] + e] = row
            want[offs[4] + e] = s0 + c
            want[offs[5] + e] = one.state_slot(r)
            for w in wants[e]:
                want[offs[6] + wi] = row + w
                wi += 1
            if feeds[e] >= 0:
                pairs += [row, feeds[e]]
            row += c
        want[offs[3] + s] = row
        want[offs[9]: offs[9] + len(pairs)] = pairs
        for g in range(2):
            sm = np.zeros(t, dtype=np.int32)
            bt = np.zeros((s, max_blocks), dtype=np.int32)
            one.fill_step(g, a_ids, a_starts, a_counts, sm, bt)
            want[offs[7] + g * t: offs[7] + (g + 1) * t] = sm
            want[offs[8] + g * s * max_blocks: offs[8] + (g + 1) * s * max_blocks] = bt.reshape(-1)
        assert n_feed == len(pairs) // 2
        assert np.array_equal(buf, want)
        for r, s0, c in zip(ids, starts, counts):
            held[r] = s0 + c
            one.release_behind(r, held[r])
        two.release_behind_all(a_ids, np.asarray([held[r] for r in ids], dtype=np.int32))
        for g in range(2):
            assert one.num_free_pages(g) == two.num_free_pages(g)
            for r in held:
                assert one.table(r, g) == two.table(r, g)
        for r in [r for r in held if rng.random() < 0.2]:
            one.free(r)
            two.free(r)
            del held[r]
        one.check()
        two.check()
    # a reservation that does not fit names its request; a wanted place outside an entry is refused
    big = CacheManager([GroupGeometry(4, 3)], 2)
    big.add(5)
    big.add(6)
    with pytest.raises(OutOfPages, match="request 6"):
        big.reserve_all(np.asarray([5, 6], dtype=np.int64), np.asarray([0, 0], dtype=np.int32),
                        np.asarray([8, 8], dtype=np.int32))
    with pytest.raises(CacheError):
        big.pack_step(np.asarray([5], dtype=np.int64), np.asarray([0], dtype=np.int32), np.asarray([2], dtype=np.int32),
                      np.asarray([1, 2], dtype=np.int32), np.asarray([-1], dtype=np.int32),
                      np.asarray([1], dtype=np.int32), np.asarray([2], dtype=np.int32), np.zeros(64, dtype=np.int32),
                      np.arange(0, 60, 6, dtype=np.int64), 2)


@pytest.mark.parametrize("page_size", [4, 16, 24, 32, 48, 64, 80, 128])
def test_a_pool_sized_for_rounded_tokens_holds_them_at_every_page_size(page_size):
    """What the replay program promises: a pool made for N tokens holds any live requests whose counts, each rounded
    up to a multiple of 64, add up to N -- also with pages of 24 or 48 tokens, which do not divide 64."""
    from atoma_infer_amd.cache.pool import CachePlan, pages_for_tokens
    plan = CachePlan(groups=[None], where={}, states={})
    live, max_tokens = 16, 16 * 64
    (pages,) = pages_for_tokens(plan, page_size, max_tokens, live)
    m = CacheManager([GroupGeometry(page_size, pages)], live)
    for r in range(live):
        m.add(r)
        m.reserve(r, 64)                   # sixteen requests of 64 rounded tokens each
    m.check()
    for r in range(live):
        m.free(r)
    # a few long requests beside short ones
    counts = [448, 320, 192, 64]
    (pages,) = pages_for_tokens(plan, page_size, sum(counts), live)
    m = CacheManager([GroupGeometry(page_size, pages)], live)
    for r, n in enumerate(counts):
        m.add(r)
        m.reserve(r, n)
    m.check()
