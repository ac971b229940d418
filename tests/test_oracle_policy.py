"""Pins for oracle/page_policy.py (CPU only).

Expected id sequences below are derived by hand from the reference's allocator rules
(lingbot_map/layers/flashinfer_cache.py:132-166 pool sizing, :496/:538 ``pop()`` takes the
last element, :507-510 anchor-then-window routing, :252-254 ``popleft`` + ``append``,
:529-553 special packing, :452-470 last page length); they are literals, not a second run
of the oracle."""
import math
import random

import pytest

from oracle.page_policy import LAYOUT_FRAME_PAGES, LAYOUT_TWO_STREAM, PagePolicy, is_keyframe


def small_policy(**kw):
    return PagePolicy(tokens_per_frame=7, num_special_tokens=3, scale_frames=1, sliding_window=2,
                      max_total_frames=6, **kw)


def test_pool_sizing_matches_reference_formula():
    p = small_policy()
    assert p.page_size == 4
    assert p.max_patch_pages == 1 + 2 + 16
    assert p.max_num_pages - p.max_patch_pages == math.ceil(6 * 3 / 4) + 16
    assert p.free_patch_pages == list(range(19))
    assert p.free_special_pages == list(range(19, 40))


# (patch page taken, anchor, window, free tail, special pages, special count, visible, last len)
TRACE = [
    (18, [18], [], [17], [39], 3, [18, 39], 3),
    (17, [18], [17], [16], [39, 38], 6, [18, 17, 39, 38], 2),
    (16, [18], [17, 16], [15], [39, 38, 37], 9, [18, 17, 16, 39, 38, 37], 1),
    (15, [18], [16, 15], [14, 17], [39, 38, 37], 12, [18, 16, 15, 39, 38, 37], 4),
    (17, [18], [15, 17], [14, 16], [39, 38, 37, 36], 15, [18, 15, 17, 39, 38, 37, 36], 3),
    (16, [18], [17, 16], [14, 15], [39, 38, 37, 36, 35], 18, [18, 17, 16, 39, 38, 37, 36, 35], 2),
]


def test_six_frame_trace_two_stream():
    p = small_policy()
    for taken, anchor, window, free_tail, special, count, visible, last in TRACE:
        plan = p.append_frame()
        assert plan.page[3] == taken  # first patch token follows the 3 specials
        p.evict_frames(1, 2)
        assert [pg[0] for pg in p.scale_patch_pages] == anchor
        assert [pg[0] for pg in p.live_window_patch_pages] == window
        assert p.free_patch_pages[-len(free_tail):] == free_tail
        assert p.all_special_pages == special
        assert p.special_token_count == count
        assert p.build_visible_page_table() == visible
        assert p.compute_last_page_len() == last
        assert p.all_pages_accounted()


def test_special_placement_crosses_page_boundary():
    p = small_policy()
    p.append_frame()
    plan = p.append_frame()  # count 3 -> one token into page 39 slot 3, two into page 38
    assert list(zip(plan.page[:3], plan.slot[:3])) == [(39, 3), (38, 0), (38, 1)]
    assert list(zip(plan.page[3:], plan.slot[3:])) == [(17, 0), (17, 1), (17, 2), (17, 3)]


def snapshot(p):
    return (list(map(list, p.scale_patch_pages)), list(map(list, p.live_window_patch_pages)),
            list(p.free_patch_pages), list(p.all_special_pages), list(p.free_special_pages),
            p.special_token_count, p.frame_count, list(p.memory_frames))


def test_non_keyframe_probe_restores_state_bit_for_bit():
    p = small_policy()
    for _ in range(6):
        p.append_frame()
        p.evict_frames(1, 2)
    before = snapshot(p)
    p._defer_eviction = True
    plan = p.append_frame()
    assert plan.page[3] == 15
    assert list(zip(plan.page[:3], plan.slot[:3])) == [(35, 2), (35, 3), (34, 0)]
    p.evict_frames(1, 2)  # deferred: no-op
    assert p.build_visible_page_table() == [18, 17, 16, 15, 39, 38, 37, 36, 35, 34]
    assert p.compute_last_page_len() == 1
    p.rollback_last_frame()
    p._defer_eviction = False
    assert snapshot(p) == before


def test_reference_sanity_check_figures():
    # lingbot_map/layers/flashinfer_cache.py:577-631
    p = PagePolicy(tokens_per_frame=262, num_special_tokens=6, scale_frames=8, sliding_window=64,
                   max_total_frames=200)
    for _ in range(100):
        p.append_frame()
        p.evict_frames(8, 64)
    assert len(p.scale_patch_pages) == 8
    assert len(p.live_window_patch_pages) == 64
    assert len(p.all_special_pages) == 3
    assert p.special_token_count == 600
    assert p.compute_last_page_len() == 88
    vis = p.build_visible_page_table()
    assert len(vis) == 8 + 64 + 3
    assert all(x < p.max_patch_pages for x in vis[:72]) and all(x >= p.max_patch_pages for x in vis[72:])
    stats = p.get_cache_stats()
    assert stats == {"frame_count": 100, "scale_pages": 8, "live_pages": 64,
                     "free_pages": p.max_patch_pages - 72, "special_tokens": 600}
    p.reset()
    assert p.frame_count == 0 and p.all_pages_accounted()


def test_rollback_in_anchor_phase_and_underflow():
    p = small_policy()
    with pytest.raises(AssertionError):
        p.rollback_last_frame()
    p.append_frame()
    p.rollback_last_frame()
    assert p.frame_count == 0 and p.special_token_count == 0 and not p.all_special_pages
    assert p.free_patch_pages == list(range(19)) and p.free_special_pages == list(range(19, 40))


def test_pool_exhaustion_asserts():
    p = small_policy()
    p._defer_eviction = True
    for _ in range(19):
        p.append_frame()
        p.evict_frames(1, 2)
    with pytest.raises(AssertionError, match="patch page pool exhausted"):
        p.append_frame()
    q = PagePolicy(tokens_per_frame=7, num_special_tokens=3, scale_frames=1, sliding_window=2, max_total_frames=1)
    n_special_slots = (math.ceil(3 / 4) + 16) * 4
    with pytest.raises(AssertionError, match="special page pool exhausted"):
        for _ in range(n_special_slots // 3 + 2):
            q.append_frame()
            q.evict_frames(1, 2)


@pytest.mark.parametrize("layout", [LAYOUT_TWO_STREAM, LAYOUT_FRAME_PAGES])
@pytest.mark.parametrize("page_size", [None, 4, 16, 5])
def test_random_scripts_conserve_pages(layout, page_size):
    rng = random.Random(1234)
    p = PagePolicy(tokens_per_frame=37, num_special_tokens=5, page_size=page_size, scale_frames=2,
                   sliding_window=3, max_total_frames=400, layout=layout, page_base=7)
    for step in range(300):
        r = rng.random()
        if r < 0.55:
            p.append_frame(); p.evict_frames(2, 3)
        elif r < 0.85:
            before = snapshot(p)
            p._defer_eviction = True
            p.append_frame(); p.evict_frames(2, 3); p.rollback_last_frame()
            p._defer_eviction = False
            assert snapshot(p) == before
        elif r < 0.95:
            p._defer_eviction = True
            p.append_frame(); p.evict_frames(2, 3)
            p._defer_eviction = False
            p.execute_deferred_eviction(2, 3)
        elif p.frame_count:
            pass
        assert p.all_pages_accounted()
        ids, lens = p.build_visible_page_table(), p.build_visible_page_lens()
        assert len(ids) == len(lens) == len(set(ids))
        assert all(1 <= n <= p.page_size for n in lens)
        kept = min(p.frame_count, 2) + min(max(p.frame_count - 2, 0), 3)
        per = 32 if layout == LAYOUT_TWO_STREAM else 37
        extra = 5 * p.frame_count if layout == LAYOUT_TWO_STREAM else 5 * (p.frame_count - kept)
        assert p.visible_tokens() == kept * per + extra


def test_frame_pages_compaction_trace():
    # tokens_per_frame 7, page 4 -> 2 pages per frame; 3 specials kept in the first page.
    p = small_policy(layout=LAYOUT_FRAME_PAGES, page_size=4)
    assert p.pages_per_frame == 2 and p.keep_pages_max == 1
    assert p.max_num_pages == 19 * 2 + 6
    top = p.max_num_pages - 1
    plan = p.append_frame(); p.evict_frames(1, 2)
    assert plan.page == [top] * 4 + [top - 1] * 3 and plan.slot == [0, 1, 2, 3, 0, 1, 2]
    p.append_frame(); p.evict_frames(1, 2)
    p.append_frame(); p.evict_frames(1, 2)
    assert p.build_visible_page_table() == [top, top - 1, top - 2, top - 3, top - 4, top - 5]
    assert p.build_visible_page_lens() == [4, 3] * 3
    p.append_frame(); p.evict_frames(1, 2)  # frame 1 leaves: keeps page top-2 with 3 tokens, frees top-3
    assert p.build_visible_page_table() == [top, top - 1, top - 4, top - 5, top - 6, top - 7, top - 2]
    assert p.build_visible_page_lens() == [4, 3, 4, 3, 4, 3, 3]
    assert p.free_patch_pages[-1] == top - 3
    plan = p.append_frame(); p.evict_frames(1, 2)  # reuses top-3 first, then top-8
    assert plan.page[0] == top - 3 and plan.page[4] == top - 8
    assert p.build_visible_page_table()[-2:] == [top - 2, top - 4]
    assert p.special_token_count == 6
    # camera-only and no-memory variants (lingbot_map/layers/attention.py:690-696)
    p.append_frame(); p.evict_frames(1, 2, camera_only=True)
    assert p.build_visible_page_lens()[-1] == 1
    n_mem = len(p.memory_frames)
    p.append_frame(); p.evict_frames(1, 2, cross_frame_special=False)
    assert len(p.memory_frames) == n_mem and p.all_pages_accounted()


def test_keyframe_rule():
    # lingbot_map/models/gct_stream.py:450
    flags = [is_keyframe(i, 1, 4) for i in range(10)]
    assert flags == [True, True, False, False, False, True, False, False, False, True]
    assert all(is_keyframe(i, 8, 1) for i in range(20))
    assert sum(is_keyframe(i, 1, 4) for i in range(320)) == 1 + 80
