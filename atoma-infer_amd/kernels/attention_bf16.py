"""bfloat16 attention over the paged cache on the matrix cores: task lists on the host, kernels per head size.

``try_attention`` runs ``attention_mfma.hip`` (compiled for the model's head size and the cache's page size on
first use) when the cache's pages hold a multiple of 16 tokens; otherwise it returns False and the caller runs the
general kernel.

The step's entries are cut into tasks of 32 query rows (row = token x query head of one KV group) against a key
range.  An entry with few tokens and many keys (a decoded token, a short portion late in a prompt) is split into
128- or 256-key chunks whose partial results a second kernel merges; everything else runs each tile against all its
keys.  The cut depends only on the entry's own start and length.  The task list is built once per step and
shared by all layers with the same grouping and window.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional, Tuple

import numpy as np
import torch

from .library import load_hip_module
from .ops import _check, _p, _stream

PAGE = 16            # the page size that the build check compiles every head size for; others on first use
CHUNK = 256          # keys per partial task, at most; fewer when few requests are split (see chunk_for)
MAX_SPLIT_TASKS = 1024
SPLIT_MAX_TOKENS = 16  # entries with at most this many tokens may be split along the keys
SPLIT_MIN_KEYS = 2 * CHUNK
SPLIT_WAVES_MIN_KEYS = 128   # a task of at least this many keys is walked by two waves, every other block each
FOUR_WAVES_MIN_KEYS = 256    # ... by four, where the launch leaves half of the GPU idle (see build_tasks)
_libs: Dict[Tuple[int, int], ctypes.CDLL] = {}


def page_ok(page_size: int) -> bool:
    """Pages that the matrix-core kernel reads: any multiple of 16 tokens (the reference's kernel takes the same:
    csrc/src/lib.rs:778-785)."""
    return page_size >= 16 and page_size % 16 == 0


def module_name(hd: int, page: int = PAGE) -> str:
    return f"attention_hd{hd}" if page == PAGE else f"attention_hd{hd}_page{page}"


def module_defines(hd: int, page: int = PAGE) -> Tuple[str, ...]:
    return (f"ATOMA_HD={hd}",) if page == PAGE else (f"ATOMA_HD={hd}", f"ATOMA_PAGE={page}")


def lib(hd: int, force_build: bool = False, page: int = PAGE) -> ctypes.CDLL:
    key = (hd, page)
    if key not in _libs or force_build:
        _libs[key] = load_hip_module(module_name(hd, page), ("attention_mfma.hip",), module_defines(hd, page),
                                     force_build=force_build)
        assert _libs[key].atoma_attention_mfma_head_size() == hd
        assert _libs[key].atoma_attention_mfma_page_size() == page
        assert _libs[key].atoma_attention_mfma_max_ksplit() == max_waves_for(hd)
        assert _libs[key].atoma_attention_mfma_max_row_tiles() == max_row_tiles_for(hd)
    return _libs[key]


def max_waves_for(hd: int) -> int:
    """Waves that may share a task for this head size: their merge must fit into the 160 KB of LDS of a CU (the
    kernel module says the same: ``atoma_attention_mfma_max_ksplit``)."""
    per_lane = -(-hd // 32) * 16 + 2
    if per_lane * 64 * 7 * 4 <= 160 * 1024:
        return 8
    return 2 if per_lane * 64 * 4 * 4 <= 160 * 1024 else 1


TWO_PIECES_MIN_KEYS = 16384     # keys from which on a wave of a prompt step works on two pieces of rows


def max_row_tiles_for(hd: int) -> int:
    """Pieces of 32 rows that a wave of a prompt step may work on against the same keys (the kernel module says the
    same: ``atoma_attention_mfma_max_row_tiles``): two where the accumulators of both fit a wave's registers."""
    return 2 if hd <= 64 else 1


# (request, KV head) pairs from which on a decoded token's keys are not cut into chunks: measured on MI355X (256 CUs),
# half as many pairs as CUs win at contexts from 2,000 to 32,000 tokens; with 64 pairs chunks win from 2,000 keys on
WHOLE_MIN_PAIRS = 128
# Fewer pairs take whole ranges too where a wave's walk is short; the walk is counted in key elements (keys times head
# size; measured at head sizes 64 and 128, 1 to 16 requests of 8 KV heads, 512 to 32,768 keys).  (pairs from, walk up to):
# 96 pairs up to 8,192 keys of head size 64 (4 to 13 % quicker than chunks), 32 up to 1,536, any number up to 1,024
# (there the second kernel costs more than the walk: 7.4 to 7.9 us against 8.9 to 10.8 at 512 keys).
WHOLE_SHORT_WALKS = ((96, 8192 * 64), (32, 1536 * 64), (1, 1024 * 64))
# keys from which on the chunks of a decoded token are 512 keys long, walked by two waves (2 to 6 % quicker steps at
# 16k to 32k tokens with 1 to 12 requests; no gain at 8k)
LONG_KEYS = 16384


# Contexts up to which the chunks of a row piece are merged by the attention kernel itself whatever the plan (the wave
# that finishes the last chunk does it; at most 18 chunks then): measured on MI355X, 0.5 to 1 us quicker than the
# merging kernel at 1,024 keys and equal at 2,048 for the pair alone, and 10 to 27 us quicker over the 16 layers of a
# decode step of 8 requests or of 1.  Beyond, the kernel merges where four waves share a chunk (decode steps, see
# ``chunk_for``: the chunks grow with the context, so the parts stay few); other plans leave the parts to the merging
# kernel, since one wave's walk over many parts costs more than the second launch.
MERGE_MAX_KEYS = 2304
MERGE_WHOLE_MAX_KEYS = 512    # with the merge in the kernel: whole ranges for few pairs only up to this many keys
MERGE_MAX_PARTS = 48          # of a row piece, where the chunks grow with the context
# (pairs from, keys beyond) which whole ranges serve such contexts at head sizes up to 64
LONG_WHOLE_PAIRS = ((512, 0), (192, 6144), (WHOLE_MIN_PAIRS, 24576))
MERGE_IN_KERNEL = True        # False: always the merging kernel (tests run both)


def merges_in_kernel(max_keys: int, waves: int = 1) -> bool:
    return MERGE_IN_KERNEL and (max_keys <= MERGE_MAX_KEYS or waves == 4)


def _long_decode_plan(pairs: int, tasks: int, max_keys: int, head_size: int) -> Optional[Tuple[int, int]]:
    """``chunk_for`` for decode steps beyond ``MERGE_MAX_KEYS`` keys whose chunks the attention kernel merges itself:
    four waves a chunk, and chunks so long that the launch has about 256 tasks, one workgroup a CU.  Measured over the
    layers of a decode step on MI355X (forward graph, 1 to 64 requests of 3,072 to 32,768 keys; 16 layers of Llama
    1B, head size 64, and 8 layers of Llama 8B, head size 128; ``tasks`` counts 256-key chunks over all KV heads):
    up to 384 tasks 256-key chunks, up to 768 512, up to 1,536 1,024, up to 2,560 2,048 (head size 64, against
    chunks walked by two waves and the merging kernel: one request of 4,096 keys 744 against 796 us, eight 933 against
    968, eight of 8,192 keys 1,135 against 1,226, one of 32,768 keys 925 against 997; head size 128: 1.5 to 6 %);
    more tasks want 1,024-key chunks at head size 64 (eight requests of 16,384 keys 1,519 against 1,586 us) and at
    wider heads the two-wave chunks with the merging kernel (None).  Whole ranges where the pairs fill the GPU: at
    head size 64 from 512 pairs, from 192 beyond 6,144 keys and from 128 beyond 24,576 (sixteen requests of 8,192
    keys: 1,661 us in chunks against 1,757 whole; twenty-four: 2,109 against 2,086)."""
    if head_size > 64:
        walk = max_keys * head_size
        if pairs >= WHOLE_MIN_PAIRS or any(pairs >= p and walk <= w for p, w in WHOLE_SHORT_WALKS):
            return 0, 8
    elif any(pairs >= p and max_keys > k for p, k in LONG_WHOLE_PAIRS):
        return 0, 8
    if tasks <= 384:
        chunk = CHUNK
    elif tasks <= 768:
        chunk = 2 * CHUNK
    elif tasks <= 1536:
        chunk = 4 * CHUNK
    elif tasks <= 2560:
        chunk = 8 * CHUNK
    elif head_size <= 64:
        chunk = 4 * CHUNK
    else:
        return None
    while max_keys > MERGE_MAX_PARTS * chunk:
        chunk *= 2
    return chunk, 4


def chunk_for(n_split: int, max_keys: int, kv_heads: int, whole_ok: bool = False, head_size: int = 64,
              ) -> Tuple[int, int]:
    """(keys per partial task, waves that share a task) for the entries of a step that are split along their keys;
    keys per task 0 means all of them: with ``whole_ok`` (a decode step, head size that allows eight waves) eight
    waves walk all keys of a (request, KV head) pair and merge in LDS, which leaves nothing to the merging kernel.
    That pays where the pairs occupy the GPU, or where a wave's share of the keys is so short that the second
    kernel costs more than the longer walk.

    A wave walks its keys one 32-key block after another, so few keys per wave shorten the chain when few requests
    decode, and long chunks save partial results (and time in the merging kernel) when many do.  Measured on
    MI355X with 2,000-token contexts and 8 KV heads: one or two requests want 128-key chunks, three to seven the
    same walked by two waves each (up to 4,096 keys: beyond, the merge of twice as many partial results costs more),
    up to about eleven 256-key chunks walked by two waves each, more requests 256-key chunks with a wave each, or 512-key
    chunks walked by two waves from 16k keys on.  The count that decides is that of 256-key tasks over all KV
    heads; ``max_keys`` is rounded up to 256.
    """
    pairs = n_split * kv_heads
    tasks = n_split * -(-max_keys // CHUNK) * kv_heads
    if whole_ok and MERGE_IN_KERNEL and max_keys > MERGE_MAX_KEYS:
        plan = _long_decode_plan(pairs, tasks, max_keys, head_size)
        if plan is not None:
            return plan
    if whole_ok and merges_in_kernel(max_keys):
        # With the chunks merged by the attention kernel itself, chunks cost no second launch, and four waves that
        # share a chunk (64 or 128 keys each, merged in LDS) shorten a wave's chain of dependent loads without more
        # partial results.  Measured over the 16 layers of a Llama 1B decode step (head size 64, 8 KV heads; 700,
        # 1,000, 1,500 and 2,049 keys; 1 to 16 requests): 256-key chunks up to 512 tasks (one request of 2,049 keys
        # 773 against 788 us a step with 128-key chunks of a wave each, four 816 against 851, eight of 1,000 keys 838
        # against 860 for whole ranges), 512-key chunks beyond (eight requests of 2,049 keys 901 against 909 us with
        # 256-key chunks of two waves, twelve of 1,500 keys 943 against 968 for whole ranges); whole ranges from 128
        # pairs on (sixteen requests of 2,049 keys 1,084 against 1,125 us) and, for the pair alone, up to 512 keys.
        if max_keys <= MERGE_WHOLE_MAX_KEYS or pairs >= WHOLE_MIN_PAIRS:
            return 0, 8
        if tasks > 544:
            return 2 * CHUNK, 4
        # few requests of up to 1,536 keys: 128-key chunks, whose parts (twelve at most) the merging wave still takes
        # in one round (one to four requests of 700 to 1,024 keys 1.5 to 2 % quicker steps at head size 64, one to
        # six at head size 128 about 1 %; with more tasks or keys the 256-key chunks are as quick or quicker)
        short_tasks = n_split * -(-max_keys // 128) * kv_heads
        if max_keys <= 1536 and short_tasks <= (400 if head_size > 64 else 200):
            return 128, 4
        return CHUNK, 4
    if whole_ok:
        walk = max_keys * head_size
        if pairs >= WHOLE_MIN_PAIRS or any(pairs >= p and walk <= w for p, w in WHOLE_SHORT_WALKS):
            return 0, 8
    if merges_in_kernel(max_keys):
        # (heads so wide that fewer than four waves may share a task; and the split entries of a prompt step)
        return (128, 1) if tasks <= 300 else (CHUNK, 2)
    if tasks <= 160:
        return 128, 1
    if tasks <= 540 and max_keys <= 4096:
        return 128, 2           # three to seven requests at 2,000 tokens: 2 to 4 % quicker steps than 256-key chunks
    if tasks <= 800:
        return CHUNK, 2
    if max_keys >= LONG_KEYS:
        return 2 * CHUNK, 2     # long contexts: half as many partial results to write and to merge
    return CHUNK, 1


def _live_pieces(rows: int, qt: int, live_tokens: int, piece: int = 32):
    """First rows of the ``piece``-row pieces of a tile that hold a live row.  Row r is token r % qt of head r // qt,
    and the tile's first ``live_tokens`` tokens exist (fewer than qt only in the last tile of an entry)."""
    if live_tokens >= qt:
        return list(range(0, rows, piece))
    out = []
    for row0 in range(0, rows, piece):
        n = min(piece, rows - row0)
        first = row0 % qt
        # rows row0 .. row0 + n - 1 hold tokens first, first + 1, ... modulo qt: live if the run starts below
        # live_tokens or wraps around to token 0
        if first < live_tokens or first + n > qt:
            out.append(row0)
    return out


def _chunk_slots(bucket_keys: int, chunk: int, window: int) -> int:
    """Partial results that a decoded token of a graph's bucket owns: one per chunk of the bucket's keys, or, with
    a window, per chunk that a window can touch wherever it lies (its first chunk is then slot 0)."""
    slots = -(-bucket_keys // chunk)
    if window > 0:
        slots = min(slots, -(-window // chunk) + 1)
    return slots


_NULL_TASK = np.asarray((-1, 0, 1, 0, 0, 0, -1, 0, 0, 0, 0, 0), dtype=np.int32)


def _tile_tasks(e: int, start: int, count: int, tok_base: int, group: int, window: int, qt: int, row_tiles: int = 1):
    """The tasks of an entry that is not split along its keys, without a loop over its tiles: (keys per group of
    four tasks, tasks [groups, 4, 12]).  A tile is ``qt`` tokens times ``group`` heads, cut into pieces of
    32 * ``row_tiles`` rows, a task each; pieces are padded to fours with empty tasks."""
    piece = 32 * row_tiles
    rows = qt * group
    pieces = -(-rows // piece)
    fours = -(-pieces // 4)
    tok0 = np.arange(0, count, qt, dtype=np.int64)                           # [tiles]
    last = np.minimum(tok0 + qt, count)
    k_end = start + last
    lo = np.maximum(0, start + tok0 - window + 1) if window > 0 else np.zeros_like(tok0)
    kb = (lo // 32) * 32
    tiles = len(tok0)
    t = np.empty((tiles, fours * 4, 12), dtype=np.int32)
    t[:] = _NULL_TASK
    row0 = piece * np.arange(pieces, dtype=np.int64)
    live = np.ones((tiles, pieces), dtype=bool)
    if int(last[-1] - tok0[-1]) < qt:                                        # the short last tile
        live[-1] = False
        live[-1, [r // piece for r in _live_pieces(rows, qt, int(last[-1] - tok0[-1]), piece)]] = True
    body = t[:, :pieces]
    vals = np.empty((tiles, pieces, 12), dtype=np.int32)
    vals[..., 0] = e
    vals[..., 1] = tok0[:, None]
    vals[..., 2] = qt
    vals[..., 3] = row0[None, :]
    vals[..., 4] = kb[:, None]
    vals[..., 5] = k_end[:, None]
    vals[..., 6] = -1
    vals[..., 7] = 0
    vals[..., 8] = tok_base
    vals[..., 9] = count
    vals[..., 10] = start
    vals[..., 11] = row_tiles
    body[live] = vals[live]
    lengths = np.repeat(k_end - kb, fours)
    return lengths, t.reshape(tiles * fours, 4, 12)


def _serpentine(n: int, kv_heads: int, compute_units: int, head_size: int = 64) -> np.ndarray:
    """The order of n groups of tasks, given longest first: the GPU takes a workgroup per (group, KV head) to its
    CUs in turn, and with head sizes up to 64 two workgroups share a CU.  So the groups of one round over all CUs
    (compute_units / kv_heads of them) keep their order and those of the next round are reversed: a CU that got a
    long group gets a short one beside it.  (A lone prompt of 2,048 tokens at Llama 1B's head shapes: 37.5 -> 32.3
    us; with less than a round there is nothing to pair, and with more than two the later workgroups go wherever a
    slot frees first, so the order stays as it is.)  Wider heads leave room for one
    workgroup a CU; the next goes to whichever CU is free first, and longest first is then the better order (head
    size 128, 2,048 tokens: 59.5 us against 71.6 reversed)."""
    if head_size > 64:
        return np.arange(n)
    if n > 2 * max(1, compute_units // max(1, kv_heads)):
        return np.arange(n)        # more than two rounds: later workgroups go where there is room, longest first is right
    per_round = max(1, compute_units // max(1, kv_heads))
    idx = np.arange(n)
    for lo in range(per_round, n, 2 * per_round):
        hi = min(lo + per_round, n)
        idx[lo:hi] = idx[lo:hi][::-1].copy()
    return idx


def build_tasks(starts: np.ndarray, counts: np.ndarray, group: int, window: int, bucket_keys: Optional[int] = None,
                vectorized: bool = True, *, kv_heads: int, max_waves: int = 2, row_tiles: int = 1,
                head_size: int = 64, compute_units: int = 256) -> Tuple[np.ndarray, tuple]:
    """Task records [n, 12] int32 (main tasks, then combine tasks), and (n_main, n_combine, n_partials, waves that
    share a task: two when a prompt tile walks many keys, else what ``chunk_for`` says for the split entries; pieces
    of 32 rows that a task which writes the output covers: ``row_tiles`` if the step has such tasks, walks at least
    ``TWO_PIECES_MIN_KEYS`` keys and two waves may share a task, else 1; whether the attention kernel merges the
    chunks itself: ``merges_in_kernel``).

    Main tasks are padded to a multiple of 4 (one workgroup runs 4) and ordered so that tasks sharing keys are
    neighbours and long tasks come first.  With ``bucket_keys`` (decode steps: one token per entry; the context
    length that the step's graph serves, in tokens) every entry is split and owns the chunk slots of that many keys,
    used or not, so all counts depend on (entries, bucket_keys) alone.
    """
    bucket = bucket_keys
    if vectorized and bucket is not None and len(counts) and int(counts.max()) == 1:
        return _build_decode_tasks(starts, group, window, bucket, kv_heads, max_waves, head_size)
    # two pieces of rows a task where the prompt tiles of the step walk long key ranges (see the kernel), and the
    # head size allows it
    longest = int((starts + counts).max()) if len(starts) else 0
    if max_waves < 2 or longest < TWO_PIECES_MIN_KEYS:
        row_tiles = 1
    qt_max = max(1, (128 * row_tiles) // group)
    piece = 32 * row_tiles
    null = (-1, 0, 1, 0, 0, 0, -1, 0, 0, 0, 0, 0)
    tok_bases = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    direct, split, combine = [], [], []
    direct_arrays = []
    n_part = 0

    def splits(e):
        first_key = max(0, int(starts[e]) - window + 1) if window > 0 else 0
        return bucket is not None or (int(counts[e]) <= SPLIT_MAX_TOKENS
                                      and int(starts[e]) + int(counts[e]) - first_key >= SPLIT_MIN_KEYS)

    split_entries = [e for e in range(len(starts)) if splits(e)]
    chunk, waves, merge = CHUNK, 1, False
    if split_entries:
        most = bucket if bucket is not None else max(int(starts[e]) + int(counts[e]) for e in split_entries)
        if bucket is not None and window > 0:
            most = min(most, window + CHUNK)
        chunk, waves = chunk_for(len(split_entries), most, kv_heads)
        waves = min(waves, max_waves)
        merge = merges_in_kernel(most)
    for e in range(len(starts)):
        start, count = int(starts[e]), int(counts[e])
        qt = min(qt_max, count)
        rows = qt * group
        do_split = splits(e)
        tail = (int(tok_bases[e]), count, start, 0)
        if vectorized and not do_split:
            lengths, groups = _tile_tasks(e, start, count, int(tok_bases[e]), group, window, qt, row_tiles)
            direct_arrays.append((lengths, groups))
            continue
        for tok0 in range(0, count, qt):
            last = min(tok0 + qt, count)
            k_end = start + last
            lo = max(0, start + tok0 - window + 1) if window > 0 else 0
            # pieces of the tile that hold at least one live row (the last tile of an entry may be short): 32 rows
            # each for tasks that leave partial results, 32 * row_tiles for those that write the output
            live = _live_pieces(rows, qt, min(qt, count - tok0), 32 if do_split else piece)
            if do_split:
                c_first, c_last = lo // chunk, (k_end - 1) // chunk
                # slot j holds chunk c_first + j
                slots = _chunk_slots(bucket, chunk, window) if bucket is not None else c_last - c_first + 1
                for row0 in live:
                    piece_index = len(combine)       # a chunk's task names the record of its row piece
                    combine.append((e, tok0, qt, row0, 0, 0, n_part, c_last - c_first + 1) + tail)
                    for j in range(slots):
                        c = c_first + j
                        if c <= c_last:
                            split.append((e, tok0, qt, row0, c * chunk, min((c + 1) * chunk, k_end), n_part + j,
                                          piece_index) + tail)
                        elif bucket is not None:
                            split.append(null)
                    n_part += slots
            else:
                kb = (lo // 32) * 32
                wave_tasks = [(e, tok0, qt, row0, kb, k_end, -1, 0) + tail[:3] + (row_tiles,) for row0 in live]
                while len(wave_tasks) % 4:
                    wave_tasks.append(null)
                direct.append((k_end - kb, wave_tasks))
    if direct_arrays:
        lengths = np.concatenate([l for l, _ in direct_arrays])
        groups = np.concatenate([g for _, g in direct_arrays])                 # [n, 4, 12]
        order = np.argsort(-lengths, kind="stable")
        head = groups[order[_serpentine(len(order), kv_heads, compute_units, head_size)]].reshape(-1, 12)
    else:
        direct.sort(key=lambda x: -x[0])
        direct = [direct[i] for i in _serpentine(len(direct), kv_heads, compute_units, head_size)]
        head = np.asarray([t for _, ws in direct for t in ws], dtype=np.int32).reshape(-1, 12)
    while len(split) % 4:
        split.append(null)
    rest = np.asarray(split + combine, dtype=np.int32).reshape(-1, 12)
    arr = np.concatenate([head, rest])
    if len(head) and int((head[:, 5] - head[:, 4]).max()) >= SPLIT_WAVES_MIN_KEYS:
        waves = 2
        # Four waves a task where the workgroups of two waves a task would fill at most half of the GPU (each then
        # becomes two): a launch lasts as long as its longest wave, and halving the walks pays while there is room
        # (prompts of 512 and 1,024 tokens at head size 64: 10.7 -> 8.8 and 17.2 -> 14.6 us; at 2,048 tokens, where
        # the GPU is full, two waves a task share their keys among more rows and win, 31 against 36 us).
        room = compute_units * (2 if head_size <= 64 else 1)
        if (max_waves >= 4 and (len(head) // 4) * kv_heads * 2 <= room
                and int((head[:, 5] - head[:, 4]).max()) >= FOUR_WAVES_MIN_KEYS):
            waves = 4
    if row_tiles > 1 and len(head):
        waves = 2                     # tasks of two pieces run in the launch of two waves a task only
    return arr, (len(head) + len(split), len(combine), n_part, waves, row_tiles if len(head) else 1, merge)


def _build_decode_tasks(starts: np.ndarray, group: int, window: int, bucket: int, kv_heads: int,
                        max_waves: int = 2, head_size: int = 64):
    """``build_tasks`` for a step in which every entry brings one token, without a Python loop over entries."""
    s = len(starts)
    starts = starts.astype(np.int64)
    k_end = starts + 1
    lo = np.maximum(0, starts - window + 1) if window > 0 else np.zeros(s, dtype=np.int64)
    row_chunks = -(-group // 32)
    # the bucket, not the step's longest request, decides between whole ranges and chunks: a graph holds one of them
    keys = bucket if window <= 0 else min(bucket, window + CHUNK)      # what a token can see
    chunk, waves = chunk_for(s, keys, kv_heads, whole_ok=max_waves >= 8, head_size=head_size)
    waves = min(waves, max_waves)
    if chunk == 0:
        whole = np.zeros((s, row_chunks, 12), dtype=np.int32)
        whole[..., 0] = np.arange(s)[:, None]
        whole[..., 2] = 1
        whole[..., 3] = 32 * np.arange(row_chunks)[None, :]
        whole[..., 4] = ((lo // 32) * 32)[:, None]
        whole[..., 5] = k_end[:, None]
        whole[..., 6] = -1
        whole[..., 8] = np.arange(s)[:, None]
        whole[..., 9] = 1
        whole[..., 10] = starts[:, None]
        return whole.reshape(-1, 12), (s * row_chunks, 0, 0, waves, 1, False)
    slots = _chunk_slots(bucket, chunk, window)
    j = np.arange(slots, dtype=np.int64)
    c_first, c_last = lo // chunk, (k_end - 1) // chunk
    c = c_first[:, None] + j[None, :]                          # [s, slots]: slot j holds chunk c_first + j
    valid = c <= c_last[:, None]
    main = np.zeros((s, row_chunks, slots, 12), dtype=np.int32)
    e = np.arange(s, dtype=np.int64)
    rc = np.arange(row_chunks, dtype=np.int64)
    v = np.broadcast_to(valid[:, None, :], (s, row_chunks, slots))
    main[..., 0] = np.where(v, e[:, None, None], -1)
    main[..., 2] = 1
    main[..., 3] = np.where(v, 32 * rc[None, :, None], 0)
    main[..., 4] = np.where(v, (c * chunk)[:, None, :], 0)
    main[..., 5] = np.where(v, np.minimum((c + 1) * chunk, k_end[:, None])[:, None, :], 0)
    part = (e[:, None, None] * row_chunks + rc[None, :, None]) * slots + j[None, None, :]
    main[..., 6] = np.where(v, part, -1)
    main[..., 7] = np.where(v, e[:, None, None] * row_chunks + rc[None, :, None], 0)      # the row piece's record
    main[..., 8] = np.where(v, e[:, None, None], 0)
    main[..., 9] = np.where(v, 1, 0)
    main[..., 10] = np.where(v, starts[:, None, None], 0)
    main = main.reshape(-1, 12)
    pad = (-len(main)) % 4
    if pad:
        filler = np.zeros((pad, 12), dtype=np.int32)
        filler[:, 0], filler[:, 2], filler[:, 6] = -1, 1, -1
        main = np.concatenate([main, filler])
    comb = np.zeros((s, row_chunks, 12), dtype=np.int32)
    comb[..., 0] = e[:, None]
    comb[..., 2] = 1
    comb[..., 3] = 32 * rc[None, :]
    comb[..., 6] = (e[:, None] * row_chunks + rc[None, :]) * slots
    comb[..., 7] = (c_last - c_first + 1)[:, None]
    comb[..., 8] = e[:, None]
    comb[..., 9] = 1
    comb[..., 10] = starts[:, None]
    arr = np.concatenate([main, comb.reshape(-1, 12)])
    return arr, (len(main), s * row_chunks, s * row_chunks * slots, waves, 1, merges_in_kernel(keys, waves))


def plan_key(group: int, window: int, kv_heads: int, hd: int):
    return ("attention_mfma_tasks", group, window, kv_heads, hd)


# Counters of the chunks that have finished, one per (row piece whose keys are cut into chunks, KV head): zeros that
# the attention kernel leaves as zeros.  One array per device, made at first use (a step's first run is never
# inside a recording); a step with more row pieces than it holds leaves its chunks to the merging kernel.
MERGE_COUNTERS = 1 << 16
_counters: Dict[torch.device, torch.Tensor] = {}


def _merge_counters(device: torch.device, needed: int) -> Optional[torch.Tensor]:
    if needed > MERGE_COUNTERS:
        return None
    t = _counters.get(device)
    if t is None:
        if torch.cuda.is_current_stream_capturing():
            return None
        t = _counters[device] = torch.zeros(MERGE_COUNTERS, dtype=torch.int32, device=device)
    return t


def try_attention(q, k_cache, v_cache, out, ctx, cache, scale, window, nh, nkv, hd) -> bool:
    """Run the fast kernels if they take this shape; False sends the caller to the general kernel."""
    page = cache.page_size
    if not page_ok(page) or hd % 16 or not 16 <= hd <= 256:
        return False
    if q.stride(0) % 8 or q.data_ptr() % 16 or out.stride(0) % 4:
        return False
    if tuple(k_cache.shape[1:]) != (nkv, page * hd) or tuple(v_cache.shape[1:]) != (nkv, page * hd):
        raise ValueError("cache tensors must be [pages, nkv, page_size * hd] tiles")
    group = nh // nkv
    plan = getattr(ctx, "plans", {}).get(plan_key(group, window, nkv, hd))
    if plan is None:
        # a caller without a step planner (a kernel test): plan here and now
        key = ("attention_tasks_adhoc", group, window, nkv, hd)
        plan = ctx.scratch.get(key)
        if plan is None:
            arr, meta = build_tasks(ctx.h_starts, ctx.h_counts, group, window, kv_heads=nkv,
                                    max_waves=max_waves_for(hd), row_tiles=max_row_tiles_for(hd))
            plan = (torch.from_numpy(arr).to(q.device), meta)
            ctx.scratch[key] = plan
    tasks, (n_main, n_comb, n_part, waves, row_tiles, merge) = plan
    ksplit = min(waves, lib(hd, page=page).atoma_attention_mfma_max_ksplit())
    part_o = part_lse = None
    if n_part:
        ws_key = ("attention_partials", nkv, hd)
        ws = ctx.scratch.get(ws_key)
        if ws is None or ws[0].shape[0] < n_part:
            ws = (torch.empty((n_part, nkv, 32, hd), dtype=torch.float32, device=q.device),
                  torch.empty((n_part, nkv, 32), dtype=torch.float32, device=q.device))
            ctx.scratch[ws_key] = ws
        part_o, part_lse = ws
    bt = cache.block_tables
    counters = _merge_counters(q.device, n_comb * nkv) if n_comb and merge else None
    _check(lib(hd, page=page).atoma_attention_mfma(_p(q), q.stride(0), _p(k_cache), _p(v_cache), _p(out), out.stride(0),
                                        _p(part_o), _p(part_lse), _p(tasks), n_main, n_comb, _p(bt), bt.shape[1],
                                        ctypes.c_float(scale), int(window), nh, nkv, ksplit, row_tiles, _p(counters),
                                        _stream()),
           "attention_mfma")
    return True
