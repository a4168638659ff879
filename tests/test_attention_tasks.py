"""The host-side task lists of the MFMA attention kernels: every (row, key) a request may see is covered exactly
once, partial results are merged from the right slots, and the vectorised decode builder equals the general one."""
import numpy as np
import pytest

from atoma_infer_amd.kernels import attention_bf16 as A


def coverage(arr, meta, starts, counts, group, window):
    n_main, n_comb, n_part, waves, tiles, merge = meta
    assert waves in (1, 2, 4, 8) and tiles in (1, 2) and (tiles == 1 or waves == 2)
    main, comb = arr[:n_main], arr[n_main:]
    assert len(comb) == n_comb and (n_main % 4 == 0 or waves == 8)    # (eight waves: one task a workgroup)
    seen = {}          # (entry, token, head) -> list of key ranges, direct
    parts = {}         # partial index -> (entry, token/head rows, key range)
    for t in main:
        e, tok0, qt, row0, kb, ke, dest, _, tok_base, count, pos0, pieces = (int(x) for x in t)
        if e < 0:
            continue
        assert tok_base == int(np.sum(counts[:e])) and count == counts[e] and pos0 == starts[e]
        assert kb % 32 == 0 and kb < ke
        # a task that writes the output covers `tiles` pieces of 32 rows, one that leaves a partial result one
        assert (max(pieces, 1) == tiles) if dest < 0 else pieces <= 1
        n_rows = 32 * max(pieces, 1)
        rows = [(tok0 + r % qt, r // qt) for r in range(row0, row0 + n_rows) if r // qt < group and tok0 + r % qt < count]
        assert rows
        if dest < 0:
            for row in rows:
                seen.setdefault((e,) + row, []).append((kb, ke))
        else:
            assert 0 <= dest < n_part and dest not in parts
            parts[dest] = (e, rows, (kb, ke))
    for t in comb:
        e, tok0, qt, row0, _, _, dest, n_parts, *_ = (int(x) for x in t)
        rows = [(tok0 + r % qt, r // qt) for r in range(row0, row0 + 32) if r // qt < group and tok0 + r % qt < counts[e]]
        for p in range(dest, dest + n_parts):
            pe, prows, rng = parts.pop(p)
            assert pe == e and prows == rows
            for row in rows:
                seen.setdefault((e,) + row, []).append(rng)
    assert not parts, "a partial result that nobody merges"
    for e in range(len(starts)):
        for tok in range(counts[e]):
            p = starts[e] + tok
            lo = max(0, p - window + 1) if window else 0
            for h in range(group):
                ranges = sorted(seen[(e, tok, h)])
                # ranges tile a span that holds every visible key, without overlap
                assert ranges[0][0] <= lo and ranges[-1][1] >= p + 1
                for (a, b), (c, d) in zip(ranges, ranges[1:]):
                    assert b == c


@pytest.mark.parametrize("seed", range(30))
def test_tasks_cover_every_visible_key_once(seed, monkeypatch):
    rng = np.random.default_rng(seed)
    s = int(rng.integers(1, 9))
    group = int(rng.choice([1, 3, 4, 8, 40]))
    window = int(rng.choice([0, 0, 50, 700]))
    counts = rng.choice([1, 1, 2, 7, 33, 150], size=s).astype(np.int32)
    starts = rng.integers(0, 2500, size=s).astype(np.int32)
    arr, meta = A.build_tasks(starts, counts, group, window, kv_heads=8)
    coverage(arr, meta, starts, counts, group, window)
    # with two pieces of rows a task (head sizes up to 64, long key ranges), by both builders
    monkeypatch.setattr(A, "TWO_PIECES_MIN_KEYS", int(rng.choice([0, 0, 1500])))
    fast, mf = A.build_tasks(starts, counts, group, window, kv_heads=8, max_waves=8, row_tiles=2)
    coverage(fast, mf, starts, counts, group, window)
    slow, ms = A.build_tasks(starts, counts, group, window, vectorized=False, kv_heads=8, max_waves=8, row_tiles=2)
    coverage(slow, ms, starts, counts, group, window)
    assert mf == ms and sorted(map(tuple, fast.tolist())) == sorted(map(tuple, slow.tolist()))


@pytest.mark.parametrize("seed", range(30))
def test_decode_builder_equals_the_general_one(seed):
    rng = np.random.default_rng(100 + seed)
    s = int(rng.integers(1, 80))
    group = int(rng.choice([1, 3, 4, 8, 40]))
    window = int(rng.choice([0, 0, 100, 700]))
    starts = rng.integers(0, 3000, size=s).astype(np.int32)
    counts = np.ones(s, dtype=np.int32)
    bucket = -(-int(starts.max() + 1) // 256) * 256
    fast, mf = A.build_tasks(starts, counts, group, window, bucket, kv_heads=8)
    slow, ms = A.build_tasks(starts, counts, group, window, bucket, vectorized=False, kv_heads=8)
    assert mf == ms
    # null tasks may differ in their unused fields; compare what the kernels read
    live = fast[:, 0] >= 0
    assert np.array_equal(live, slow[:, 0] >= 0)
    assert np.array_equal(fast[live], slow[live])
    coverage(fast, mf, starts, counts, group, window)
    # sizes depend on (entries, bucket) alone
    other = rng.integers(0, bucket, size=s).astype(np.int32)
    assert A.build_tasks(other, counts, group, window, bucket, kv_heads=8)[1] == mf


@pytest.mark.parametrize("seed", range(8))
def test_long_contexts(seed):
    """Contexts of tens of thousands of keys: longer chunks, the same coverage, both builders alike."""
    rng = np.random.default_rng(500 + seed)
    s = int(rng.integers(1, 12))
    group, window = int(rng.choice([1, 4, 8])), int(rng.choice([0, 0, 9000]))
    starts = rng.integers(15000, 40000, size=s).astype(np.int32)
    counts = np.ones(s, dtype=np.int32)
    bucket = -(-int(starts.max() + 1) // 256) * 256
    # where at most two waves may share a task (wide heads): two-wave chunks, left to the merging kernel
    fast, mf = A.build_tasks(starts, counts, group, window, bucket, kv_heads=8, max_waves=2)
    slow, ms = A.build_tasks(starts, counts, group, window, bucket, vectorized=False, kv_heads=8, max_waves=2)
    assert mf == ms
    live = fast[:, 0] >= 0
    assert np.array_equal(live, slow[:, 0] >= 0) and np.array_equal(fast[live], slow[live])
    coverage(fast, mf, starts, counts, group, window)
    seen = min(bucket, window + 256) if window else bucket       # keys a token can see
    if seen >= A.LONG_KEYS and s * -(-seen // 256) * 8 > 800:
        spans = fast[live][:, 5] - fast[live][:, 4]
        assert int(spans.max()) == 512 and mf[3] == 2 and not mf[5]
    # where eight may: four waves a chunk, the chunks the longer the more tasks there are, merged by the kernel
    wide, mw = A.build_tasks(starts, counts, group, window, bucket, kv_heads=8, max_waves=8)
    coverage(wide, mw, starts, counts, group, window)
    assert mw[3] == 4 and mw[5] is True
    spans = wide[wide[:, 0] >= 0][: mw[0]][:, 5] - wide[wide[:, 0] >= 0][: mw[0]][:, 4]
    assert int(spans.max()) in (256, 512, 1024, 2048) and -(-seen // int(spans.max())) <= A.MERGE_MAX_PARTS
    # a portion of a prompt beside them
    counts2 = counts.copy()
    counts2[0] = 40
    arr, meta = A.build_tasks(starts, counts2, group, window, kv_heads=8)
    coverage(arr, meta, starts, counts2, group, window)


@pytest.mark.parametrize("seed", range(10))
def test_whole_ranges_for_many_decoding_requests(seed):
    """Enough (request, KV head) pairs to fill the GPU: a decoded token's keys are one task for eight waves, and
    nothing is left to merge."""
    rng = np.random.default_rng(900 + seed)
    s = int(rng.integers(24, 100))
    group, window = int(rng.choice([1, 4, 8])), int(rng.choice([0, 0, 300]))
    starts = rng.integers(0, 2300, size=s).astype(np.int32)
    counts = np.ones(s, dtype=np.int32)
    bucket = -(-int(starts.max() + 1) // 256) * 256
    arr, meta = A.build_tasks(starts, counts, group, window, bucket, kv_heads=8, max_waves=8)
    assert meta == (s * -(-group // 32), 0, 0, 8, 1, False)
    coverage(arr, meta, starts, counts, group, window)
    # a head size that does not allow eight waves, or few pairs with many keys to walk: chunks as before
    assert A.build_tasks(starts, counts, group, window, bucket, kv_heads=8, max_waves=2)[1][1] > 0
    far = np.full(8, 2999, dtype=np.int32)
    assert A.build_tasks(far, counts[:8], group, 0, 3072, kv_heads=8, max_waves=8)[1][1] > 0
    assert A.build_tasks(far, counts[:8], group, 0, 3072, kv_heads=8, max_waves=8, head_size=128)[1][1] > 0
    # few pairs with few keys to walk: whole ranges again (the second kernel would cost more than the walk)
    near = np.full(8, 500, dtype=np.int32)
    arr2, meta2 = A.build_tasks(near, counts[:8], group, 0, 512, kv_heads=8, max_waves=8)
    assert meta2 == (8 * -(-group // 32), 0, 0, 8, 1, False)
    coverage(arr2, meta2, near, counts[:8], group, 0)
    assert A.build_tasks(near + 500, counts[:8], group, 0, 1024, kv_heads=8, max_waves=8)[1][1] > 0
    # contexts whose chunks the attention kernel merges itself: four waves share a chunk of 256 keys, of 512 where
    # there are many; whole ranges for short contexts and from sixteen requests of 8 KV heads on; a wave a chunk for
    # wide heads with few tasks, and where fewer than four waves may share a task
    assert A.chunk_for(1, 2048, 8, whole_ok=True, head_size=64) == (256, 4)
    assert A.chunk_for(8, 2048, 8, whole_ok=True, head_size=64) == (256, 4)
    assert A.chunk_for(8, 2304, 8, whole_ok=True, head_size=64) == (512, 4)
    assert A.chunk_for(12, 2048, 8, whole_ok=True, head_size=128) == (512, 4)
    assert A.chunk_for(16, 2048, 8, whole_ok=True, head_size=64) == (0, 8)
    assert A.chunk_for(4, 512, 8, whole_ok=True, head_size=64) == (0, 8)
    assert A.chunk_for(1, 2048, 8, whole_ok=True, head_size=128) == (256, 4)
    assert A.chunk_for(2, 1024, 8, whole_ok=True, head_size=64) == (128, 4)
    assert A.chunk_for(4, 1024, 8, whole_ok=True, head_size=64) == (256, 4)
    assert A.chunk_for(4, 1024, 8, whole_ok=True, head_size=128) == (128, 4)
    assert A.chunk_for(1, 1792, 8, whole_ok=True, head_size=64) == (256, 4)
    assert A.chunk_for(1, 2048, 8, whole_ok=False, head_size=64) == (128, 1)
    # longer contexts: four waves a chunk and chunks so long that about 256 tasks are left, merged by the kernel
    assert A.chunk_for(1, 4096, 8, whole_ok=True, head_size=64) == (256, 4)
    assert A.chunk_for(4, 4096, 8, whole_ok=True, head_size=64) == (512, 4)
    assert A.chunk_for(8, 4096, 8, whole_ok=True, head_size=128) == (1024, 4)
    assert A.chunk_for(8, 8192, 8, whole_ok=True, head_size=64) == (2048, 4)
    assert A.chunk_for(1, 32768, 8, whole_ok=True, head_size=64) == (1024, 4)
    assert A.chunk_for(8, 16384, 8, whole_ok=True, head_size=64) == (1024, 4)
    assert A.chunk_for(16, 8192, 8, whole_ok=True, head_size=64) == (1024, 4)
    # (a row piece's parts stay few however long the context)
    chunk, waves = A.chunk_for(1, 131072, 8, whole_ok=True, head_size=64)
    assert waves == 4 and 131072 <= A.MERGE_MAX_PARTS * chunk
    assert A.merges_in_kernel(131072, 4) and not A.merges_in_kernel(131072, 2) and A.merges_in_kernel(2048, 2)
    # whole ranges where the pairs fill the GPU
    assert A.chunk_for(64, 4096, 8, whole_ok=True, head_size=64) == (0, 8)
    assert A.chunk_for(24, 8192, 8, whole_ok=True, head_size=64) == (0, 8)
    assert A.chunk_for(24, 4096, 8, whole_ok=True, head_size=64) == (1024, 4)
    assert A.chunk_for(16, 32768, 8, whole_ok=True, head_size=64) == (0, 8)
    assert A.chunk_for(16, 8192, 8, whole_ok=True, head_size=128) == (0, 8)
    assert A.chunk_for(12, 4096, 8, whole_ok=True, head_size=128) == (0, 8)
    # wide heads with many tasks: two waves a chunk and the merging kernel, as where fewer than four waves may share
    assert A.chunk_for(8, 32768, 8, whole_ok=True, head_size=128) == (512, 2)
    assert A.chunk_for(12, 32768, 8, whole_ok=False, head_size=64)[1] <= 2
    # the merge of the waves' shares must fit the 160 KB of LDS of a CU: eight waves up to heads of 160, two beyond
    assert A.max_waves_for(64) == 8 and A.max_waves_for(128) == 8 and A.max_waves_for(160) == 8
    assert A.max_waves_for(176) == 2 and A.max_waves_for(256) == 2


@pytest.mark.parametrize("seed", range(20))
def test_tile_builder_equals_the_general_one(seed):
    """Entries that are not split along their keys are planned without a loop over their tiles; the plain loop
    gives the same tasks."""
    rng = np.random.default_rng(500 + seed)
    s = int(rng.integers(1, 7))
    group = int(rng.choice([1, 3, 4, 8, 40, 130]))
    window = int(rng.choice([0, 0, 50, 700]))
    counts = rng.choice([1, 1, 2, 7, 33, 150, 600], size=s).astype(np.int32)
    starts = rng.integers(0, 2500, size=s).astype(np.int32)
    fast, mf = A.build_tasks(starts, counts, group, window, kv_heads=8)
    slow, ms = A.build_tasks(starts, counts, group, window, vectorized=False, kv_heads=8)
    assert mf[1:] == ms[1:]
    live = lambda arr, meta: sorted(map(tuple, arr[:meta[0]][arr[:meta[0], 0] >= 0].tolist()))
    assert live(fast, mf) == live(slow, ms)
    assert np.array_equal(fast[mf[0]:], slow[ms[0]:])
    coverage(fast, mf, starts, counts, group, window)


def test_a_window_far_into_a_context_owns_few_slots():
    """A decoded token behind a window sees a few chunks wherever it stands: its request owns slots for those,
    not for every chunk of its context."""
    starts = np.asarray([100_000, 70_001, 5], dtype=np.int32)
    counts = np.ones(3, dtype=np.int32)
    bucket = -(-100_001 // 256) * 256
    for builder in (True, False):
        arr, meta = A.build_tasks(starts, counts, 4, 1000, bucket, vectorized=builder, kv_heads=8, max_waves=2)
        coverage(arr, meta, starts, counts, 4, 1000)
        assert meta[2] <= 3 * (1000 // 128 + 2) and meta[0] <= meta[2] + 3
    without, meta_all = A.build_tasks(starts, counts, 4, 0, bucket, kv_heads=8, max_waves=2)
    assert meta_all[2] > 500


def test_long_and_short_groups_meet_on_a_cu():
    """Groups come longest first; every second round over the CUs is reversed, so that the workgroups which share a
    CU's slots add up to about the same number of keys."""
    order = A._serpentine(7, 8, 32)             # 4 groups a round
    assert order.tolist() == [0, 1, 2, 3, 6, 5, 4]
    assert A._serpentine(10, 8, 32).tolist() == list(range(10))            # more than two rounds: as it was
    assert A._serpentine(5, 8, 256).tolist() == [0, 1, 2, 3, 4]            # less than a round: as it was
    assert A._serpentine(7, 8, 32, head_size=128).tolist() == list(range(7))        # one workgroup a CU: as it was
    for n, kv, cus in ((64, 8, 256), (7, 1, 4), (100, 3, 64)):
        assert sorted(A._serpentine(n, kv, cus).tolist()) == list(range(n))
    # a lone prompt of 2,048 tokens, 8 KV heads, 256 CUs: the keys of groups i and 63 - i... sum to the same
    arr, meta = A.build_tasks(np.asarray([0], dtype=np.int32), np.asarray([2048], dtype=np.int32), 4, 0, kv_heads=8)
    spans = (arr[: meta[0], 5] - arr[: meta[0], 4]).reshape(-1, 4).max(axis=1)
    assert len(spans) == 64
    sums = spans[:32] + spans[32:]
    assert sums.max() - sums.min() <= 32
    coverage(arr, meta, np.asarray([0]), np.asarray([2048]), 4, 0)


def test_four_waves_a_task_where_two_would_leave_half_of_the_gpu_idle():
    """A prompt whose tiles, at two waves a task, make no more workgroups than half of what the GPU holds is walked
    by four waves a task (each workgroup becomes two); a prompt that fills the GPU keeps two, and so does a head size
    whose merge of four waves' results does not fit."""
    one = lambda n, **kw: A.build_tasks(np.asarray([0], dtype=np.int32), np.asarray([n], dtype=np.int32), 4, 0,
                                        kv_heads=8, **kw)[1]
    assert one(1024, max_waves=8)[3] == 4 and one(512, max_waves=8)[3] == 4
    assert one(2048, max_waves=8)[3] == 2                       # 512 workgroups: the GPU is full
    assert one(1024, max_waves=2)[3] == 2                       # the head size allows two at most
    assert one(1024, max_waves=8, head_size=128)[3] == 2        # one workgroup a CU: 256 are a full round
    assert one(512, max_waves=8, head_size=128)[3] == 4
    assert one(100, max_waves=8)[3] == 1                        # short walks: a wave a task
