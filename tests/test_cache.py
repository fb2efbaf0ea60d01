"""The cache's bookkeeping: no slot or page lost, held twice or freed twice; windowed groups
give pages back; a step that does not fit changes nothing."""
import random

import pytest
import torch

from agave_amd.cache import (PAGE, CacheError, GroupKey, GroupPages, KVCache, OutOfPages, OutOfSlots, PagePool,
                             SlotTable, StateNeed)


def test_page_pool_alloc_free():
    pool = PagePool(4)
    got = [pool.alloc() for _ in range(4)]
    assert sorted(got) == [0, 1, 2, 3] and pool.n_free == 0
    with pytest.raises(OutOfPages):
        pool.alloc()
    pool.free(2)
    with pytest.raises(CacheError):
        pool.free(2)                        # freed twice
    with pytest.raises(CacheError):
        pool.free(9)
    assert pool.alloc() == 2                # used again
    for p in got:
        pool.free(p)
    assert pool.n_free == 4


def test_slot_table():
    st = SlotTable(2)
    a, b = st.alloc(), st.alloc()
    assert {a, b} == {0, 1}
    with pytest.raises(OutOfSlots):
        st.alloc()
    st.free(a)
    with pytest.raises(CacheError):
        st.free(a)
    assert st.alloc() == a and st.length[a] == 0


def _cache(window=None, n_pages=8, slots=3, ctx=512):
    full, win = GroupKey(None, 1, 8), GroupKey(window, 1, 8)
    needs = {0: win, 1: full, 2: win} if window else {0: full, 1: full}
    return KVCache(needs, {}, slots, {k: n_pages for k in set(needs.values())}, torch.float32, None, ctx)


def test_full_group_tables_and_release():
    c = _cache()
    s = c.alloc_slot()
    pos0, plans = c.plan_step([s], [70])
    assert pos0 == [0] and plans[0].base == [0] and len(plans[0].rows[0]) == 2
    c.commit_step([s], [70])
    assert c.length(s) == 70
    pos0, plans = c.plan_step([s], [1])
    assert pos0 == [70] and len(plans[0].rows[0]) == 2          # position 70 is in page 1: nothing new
    c.commit_step([s], [1])
    for _ in range(57):
        c.plan_step([s], [1]); c.commit_step([s], [1])
    assert c.length(s) == 128
    _, plans = c.plan_step([s], [1])
    assert len(plans[0].rows[0]) == 3
    c.commit_step([s], [1])
    c.free_slot(s)
    assert c.groups[0].pool.n_free == 8 and c.slots.n_free == 3
    with pytest.raises(CacheError):
        c.free_slot(s)


def test_window_group_gives_pages_back_and_keeps_reach():
    W = 100
    c = _cache(window=W, n_pages=16, ctx=1024)
    gi = [i for i, k in enumerate(c.group_keys) if k.window == W][0]
    g = c.groups[gi]
    s = c.alloc_slot()
    c.plan_step([s], [500]); c.commit_step([s], [500])
    held = g.held(s)
    # a query at position >= 500 reaches back to 500 - W + 1 = 401 -> page 6
    assert min(held) == 401 // PAGE and max(held) == 499 // PAGE
    for step in range(200):
        L = c.length(s)
        _, plans = c.plan_step([s], [1])
        base, row = plans[gi].base[0], plans[gi].rows[0]
        assert base == max(0, L - W + 1) // PAGE
        assert base + len(row) - 1 == L // PAGE
        assert len(set(row)) == len(row)
        c.commit_step([s], [1])
        assert len(g.held(s)) <= W // PAGE + 2
    c.free_slot(s)
    assert all(x.pool.n_free == x.pool.n_pages for x in c.groups)


def test_step_that_does_not_fit_changes_nothing():
    c = _cache(n_pages=4)
    a, b = c.alloc_slot(), c.alloc_slot()
    with pytest.raises(OutOfPages):
        c.plan_step([a, b], [130, 130])            # 3 + 3 pages > 4
    assert c.groups[0].pool.n_free == 4 and c.groups[0].held(a) == {}
    c.plan_step([a, b], [64, 128]); c.commit_step([a, b], [64, 128])
    with pytest.raises(CacheError, match="context"):
        c.plan_step([a], [512])
    with pytest.raises(CacheError, match="twice"):
        c.plan_step([a, a], [1, 1])
    with pytest.raises(CacheError):
        c.plan_step([2], [1])                      # slot not held


def test_random_traffic_never_loses_or_doubles_a_page():
    rnd = random.Random(0)
    c = _cache(window=70, n_pages=40, slots=5, ctx=600)
    live = {}
    for _ in range(400):
        if live and rnd.random() < 0.15:
            s = rnd.choice(list(live))
            c.free_slot(s); del live[s]
        elif len(live) < 5 and rnd.random() < 0.3:
            s = c.alloc_slot()
            assert s not in live
            live[s] = 0
        elif live:
            s = rnd.choice(list(live))
            n = rnd.choice([1, 1, 1, 5, 64, 130])
            try:
                c.plan_step([s], [n])
            except (OutOfPages, CacheError):
                continue
            c.commit_step([s], [n]); live[s] += n
            assert c.length(s) == live[s]
        for g in c.groups:
            held = [p for s in range(5) for p in g.held(s).values()]
            assert len(held) == len(set(held))                       # no page held twice
            assert len(held) + g.pool.n_free == g.pool.n_pages       # none lost
    for s in list(live):
        c.free_slot(s)
    assert all(g.pool.n_free == g.pool.n_pages for g in c.groups) and c.slots.n_free == 5


def test_groups_and_state():
    full, win = GroupKey(None, 2, 16), GroupKey(8, 2, 16)
    c = KVCache({0: win, 1: win, 2: full, 3: win}, {1: StateNeed((3, 4))}, 2, {full: 4, win: 6},
                torch.float32, torch.device("cpu"), 256)
    assert c.group_keys == [win, full]
    assert c.k_store[0].shape == (3, 6, 2, PAGE, 16) and c.v_store[0].shape == (3, 6, 2, 16, PAGE)
    assert c.k_store[1].shape == (1, 4, 2, PAGE, 16)
    assert c.index_in_group == {0: 0, 1: 1, 2: 0, 3: 2}
    k, v, packed = c.pages_of(3)
    assert k.data_ptr() == c.k_store[0][2].data_ptr() and not packed     # 32-bit pages are kept row by row
    s = c.alloc_slot()
    c.state[1][s].fill_(5.0)
    c.free_slot(s)
    assert c.alloc_slot() == s and float(c.state[1][s].abs().sum()) == 0.0    # zeroed when taken again


def test_table_width():
    g = GroupPages(GroupKey(1024, 1, 8), 64, 2)
    assert g.table_width(4096) == 17 and g.table_width(512) == 8
    assert GroupPages(GroupKey(None, 1, 8), 64, 2).table_width(4096) == 64


def test_pool_sizes_follow_each_group_reach():
    from agave_amd.cache import pages_in_reach, pool_pages
    # all keys: the whole context of every slot
    assert pool_pages(None, 8, 131072, 4096) == 8 * 2048
    # a window of 1024 and pieces of 4096: 1024 + 4095 positions touch at most 81 + 1 pages
    assert pages_in_reach(1024, 131072, 4096) == (1024 + 4096 - 1 + 62) // 64 + 1 == 81
    assert pool_pages(1024, 8, 131072, 4096) == 8 * 81
    # never more than the context itself, and a piece is never longer than the context
    assert pool_pages(1024, 8, 4096, 4096) == 8 * 64 and pool_pages(1024, 3, 512, 99999) == 3 * 8
    # decoding only: the window's reach
    assert pages_in_reach(1024, 131072, 1) == 17 and pages_in_reach(16, 64, 1) == 1
    # every alignment of a step inside its pages fits the bound, and one alignment reaches it
    for window, piece in ((16, 1), (70, 5), (100, 130), (1024, 64)):
        bound = pages_in_reach(window, 10 ** 6, piece)
        spans = []
        for pos0 in range(0, 4 * 64 + window):
            lo = max(0, pos0 - window + 1) // PAGE
            spans.append((pos0 + piece - 1) // PAGE - lo + 1)
        assert max(spans) == bound


def test_published_sizes_fit_one_gpu_at_the_whole_context():
    """Gemma 3 27B at 131,072 positions and 8 slots: the windowed layers' share does not grow
    with the context."""
    from agave_amd.cache import pool_pages
    layers, pattern, nkv, hd, window = 62, 6, 16, 128, 1024
    n_window = sum(1 for i in range(layers) if (i + 1) % pattern)
    page_bytes = 2 * 64 * nkv * hd * 2                       # K and V, bfloat16
    full = (layers - n_window) * pool_pages(None, 8, 131072, 4096) * page_bytes
    win = n_window * pool_pages(window, 8, 131072, 4096) * page_bytes
    assert n_window == 52 and full == 10 * 16384 * page_bytes
    assert win == 52 * 8 * 81 * page_bytes and (full + win) / 2 ** 30 < 100
    same_as_full = layers * pool_pages(None, 8, 131072, 4096) * page_bytes
    assert same_as_full / 2 ** 30 > 490


def test_a_step_in_pieces_is_checked_as_a_whole():
    from agave_amd.engine.step import split_pieces
    assert split_pieces([5, 300, 128, 129], 128) == [[0, 128, 0, 128], [0, 128, 0, 0], [5, 44, 128, 1]]
    assert split_pieces([7], 128) == [[7]] and split_pieces([256], 128) == [[128], [128]]
    W = 70
    full, win = GroupKey(None, 1, 8), GroupKey(W, 1, 8)
    # the windowed pool holds the window's reach plus a piece of 128 for two slots, no more
    from agave_amd.cache import pool_pages
    n_win = pool_pages(W, 2, 2048, 128)
    c = KVCache({0: win, 1: full}, {}, 2, {win: n_win, full: 40}, torch.float32, None, 2048)
    a, b = c.alloc_slot(), c.alloc_slot()
    with pytest.raises(OutOfPages):
        c.check_pieces([a, b], [[1500, 900]])                  # as one piece the windowed pool is too small
    pieces = split_pieces([1500, 900], 128)
    c.check_pieces([a, b], pieces)
    for counts in pieces:                                      # and the pieces do run, one after another
        idx = [i for i, n in enumerate(counts) if n]
        c.plan_step([[a, b][i] for i in idx], [counts[i] for i in idx])
        c.commit_step([[a, b][i] for i in idx], [counts[i] for i in idx])
    assert c.length(a) == 1500 and c.length(b) == 900
    with pytest.raises(CacheError, match="context"):
        c.check_pieces([a], split_pieces([600], 128))
    # a group that needs all keys counts every piece: 24 of its 40 pages are held, 1100 positions need 18
    c.free_slot(b)
    b = c.alloc_slot()
    free_before = [g.pool.n_free for g in c.groups]
    with pytest.raises(OutOfPages):
        c.check_pieces([b], split_pieces([1100], 128))
    assert [g.pool.n_free for g in c.groups] == free_before and c.length(b) == 0


def test_a_table_narrower_than_a_step_s_reach_is_refused_on_the_host():
    """The prefill kernel indexes a row of page ids by page index; the wrapper refuses a table whose
    rows do not cover what the step's queries reach, before anything is launched."""
    from agave_amd.ops.attention_mfma import check_table_reach
    check_table_reach([0, 130], [200, 1], None, [0, 0], 4)               # pages 0..3 and 0..2
    check_table_reach([1000], [70], 100, [14], 3)                        # reach 901..1069: pages 14..16
    with pytest.raises(ValueError, match="columns"):
        check_table_reach([0], [257], None, [0], 4)                      # page 4 is outside 4 columns
    with pytest.raises(ValueError, match="reach back"):
        check_table_reach([1000], [70], 100, [15], 3)                    # the row starts after page 14
    with pytest.raises(ValueError, match="reach back"):
        check_table_reach([1000], [1], None, [3], 64)                    # all keys: the row must start at page 0


@pytest.mark.parametrize("pos0,n_new,window,blk_len", [([0], [2048], 1024, 64), ([0], [2048], None, 64),
                                                       ([5, 0, 100], [1, 70, 300], 70, 32), ([4000], [200], 1500, 64),
                                                       ([0, 0, 0], [33, 4096, 640], 1024, 64)])
def test_the_items_of_a_prefill_step_cover_every_block_and_page_once(pos0, n_new, window, blk_len):
    """The host cuts a step of several tokens per sequence into items (a block of positions and a
    run of the pages it sees): together they cover each block's reach exactly once, the pieces of a
    block are runs that follow each other, the list starts with the largest, and every token knows
    how many pieces its block has."""
    import numpy as np
    from agave_amd.ops.attention_mfma import ITEM_MAX_PIECES, plan_prefill_items
    items, tok_pieces, max_pieces, max_pages = plan_prefill_items(pos0, n_new, window, blk_len, 4, 8, 256)
    assert items.dtype == np.int32 and items.shape[1] == 6 and 1 <= max_pieces <= ITEM_MAX_PIECES
    assert list(items[:, 3]) == sorted(items[:, 3], reverse=True) and max_pages == items[:, 3].max()
    starts = np.concatenate([[0], np.cumsum(n_new)])
    seen = {}
    for b, blk0, pg0, npg, piece, pieces in items.tolist():
        assert npg >= 1 and 0 <= piece < pieces <= max_pieces
        seen.setdefault((b, blk0), []).append((piece, pg0, npg, pieces))
    for b, (p0, n) in enumerate(zip(pos0, n_new)):
        for blk0 in range(0, n, blk_len):
            first, last = p0 + blk0, p0 + min(n, blk0 + blk_len) - 1
            lo = max(0, first - window + 1) if window else 0
            got = sorted(seen.pop((b, blk0)))
            assert [g[0] for g in got] == list(range(got[0][3])) and all(g[3] == got[0][3] for g in got)
            assert got[0][1] == lo // 64 and got[-1][1] + got[-1][2] - 1 == last // 64
            for x, y in zip(got, got[1:]):
                assert x[1] + x[2] == y[1]                        # runs that follow each other
            assert (tok_pieces[starts[b] + blk0:starts[b] + min(n, blk0 + blk_len)] == got[0][3]).all()
    assert not seen and len(tok_pieces) == sum(n_new)


def test_the_decode_attention_s_split_plan():
    """The number of splits stays within what the kernels and the merge take, whatever the sizes,
    and follows the measured rules at the sizes they were measured at."""
    from agave_amd.ops.attention_mfma import split_plan, MAX_SPLITS
    for hd in (0, 64, 128, 256):
        for span in (1, 2, 5, 17, 40, 63, 64, 121, 512, 2048):
            for units in (1, 4, 8, 32, 33, 64, 100, 128, 256, 1000):
                splits, per = split_plan(span, units, hd)
                limit = MAX_SPLITS if hd else 256        # (the general kernel's merge takes 256 shares)
                assert 1 <= splits <= min(span, limit) and per * splits >= span, (hd, span, units)
    # 17 pages in reach, head size 256: a batch of 1, 8, 16, 17, 24 and 32 sequences of the 4B sizes (4 kv heads)
    assert [split_plan(17, b * 4, 256)[0] for b in (1, 8, 16, 17, 24, 32)] == [12, 5, 3, 3, 2, 1]
    # 500 pages: six splits at 32 units, and a launch that would leave half the chip idle is split further
    assert split_plan(500, 32, 256)[0] == 6 and split_plan(500, 128, 256)[0] == 2
