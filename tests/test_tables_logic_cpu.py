"""The table state machine the HIP kernel runs (csrc/tables_logic.h), compiled for the host
and replayed against the oracle policy: page ids, lengths, append rows and visible rows must
match bit for bit after every operation.  CPU only."""
import ctypes as C
import os
import random
import subprocess
import tempfile

import numpy as np
import pytest

from oracle.page_policy import LAYOUT_FRAME_PAGES, LAYOUT_TWO_STREAM, PagePolicy

HERE = os.path.dirname(os.path.abspath(__file__))
OP_RESET, OP_ROLLBACK, OP_APPEND, OP_EVICT, OP_PLAN = 1, 2, 4, 8, 16


class Geom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("layout", "tokens_per_frame", "num_special_tokens", "page_size",
                                         "scale_frames", "patch_pages", "special_pages", "memory_frames",
                                         "pages_per_stream")]


class Op(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("ops", "sliding_window", "keep_tokens", "self_tokens", "q_begin",
                                         "kv_row_begin", "expect_kv_tokens", "page_out_begin")]


@pytest.fixture(scope="module")
def host_lib():
    d = tempfile.mkdtemp(prefix="lbm_tables_host_")
    so = os.path.join(d, "tables_host.so")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-Wall", "-Werror",
                           "-o", so, os.path.join(HERE, "native", "tables_host.cpp")])
    lib = C.CDLL(so)
    lib.lbm_tables_words_host.restype = C.c_longlong
    return lib


class HostTables:
    """Drives the host build the way the manager drives the kernel, for one or more streams."""

    def __init__(self, lib, pol: PagePolicy, n_streams=1, max_total_frames=0):
        self.lib, self.pol, self.n = lib, pol, n_streams
        two = pol.layout == LAYOUT_TWO_STREAM
        self.g = Geom(0 if two else 1, pol.tokens_per_frame, pol.num_special_tokens, pol.page_size, pol.scale_frames,
                      pol.max_patch_pages, pol.max_special_pages, 0 if two else max_total_frames, pol.max_num_pages)
        self.words = lib.lbm_tables_words_host(C.byref(self.g))
        assert self.words > 0
        self.tables = np.zeros(n_streams * self.words, dtype=np.int32)
        self.rows_cap, self.pages_cap = 4096, 1024
        self.append_rows = np.full(n_streams * pol.tokens_per_frame, -7, dtype=np.int32)
        self.kv_rows = np.full(n_streams * self.rows_cap, -9, dtype=np.int32)
        self.ids = np.zeros(n_streams * self.pages_cap, dtype=np.int32)
        self.lens = np.zeros(n_streams * self.pages_cap, dtype=np.int32)
        self.step([{"ops": OP_RESET}] * n_streams)

    def step(self, per_stream, append=False, plan=False):
        ops = (Op * self.n)()
        for b, d in enumerate(per_stream):
            ops[b].q_begin = b * self.pol.tokens_per_frame
            ops[b].kv_row_begin = b * self.rows_cap
            ops[b].page_out_begin = b * self.pages_cap
            for k, v in d.items():
                setattr(ops[b], k, v)
        p = lambda a: a.ctypes.data_as(C.c_void_p)
        rc = self.lib.lbm_tables_step_host(p(self.tables), C.byref(self.g), self.n, ops,
                                           p(self.append_rows) if append else None,
                                           p(self.kv_rows) if plan else None,
                                           p(self.ids) if plan else None, p(self.lens) if plan else None)
        assert rc == 0

    def hdr(self, b=0):
        return self.tables[b * self.words: b * self.words + 16]

    def visible(self, expect, b=0, self_tokens=0):
        self.step([{"ops": OP_PLAN if i == b else 0, "expect_kv_tokens": expect, "self_tokens": self_tokens}
                   for i in range(self.n)], plan=True)
        n_pages = int(self.hdr(b)[12])
        lo = b * self.pages_cap
        rows = self.kv_rows[b * self.rows_cap: b * self.rows_cap + expect].tolist()
        return self.ids[lo:lo + n_pages].tolist(), self.lens[lo:lo + n_pages].tolist(), rows


def oracle_rows(pol):
    rows = []
    S = pol.page_size
    for p, n in zip(pol.build_visible_page_table(), pol.build_visible_page_lens()):
        rows += [p * 2 * S + s for s in range(n)]
    return rows


def check_same(ht: HostTables, pol: PagePolicy, b=0):
    ids, lens, rows = ht.visible(pol.visible_tokens(), b)
    assert ids == pol.build_visible_page_table()
    assert lens == pol.build_visible_page_lens()
    assert rows == oracle_rows(pol)
    h = ht.hdr(b)
    assert h[10] == 0, f"device error word {h[10]}"
    assert h[0] == pol.frame_count and h[4] == len(pol.free_patch_pages) and h[7] == pol.special_token_count
    assert h[11] == pol.visible_tokens()
    # free lists are compared as sequences: recycling order is part of the policy
    L0 = 16
    free = ht.tables[b * ht.words + L0: b * ht.words + L0 + h[4]].tolist()
    assert free == pol.free_patch_pages
    if pol.layout == LAYOUT_TWO_STREAM:
        fs0 = b * ht.words + L0 + pol.max_patch_pages
        assert ht.tables[fs0: fs0 + h[5]].tolist() == pol.free_special_pages


def test_six_frame_trace_on_host_build(host_lib):
    pol = PagePolicy(7, 3, None, 1, 2, max_total_frames=6)
    ht = HostTables(host_lib, pol)
    expected_visible = [[18, 39], [18, 17, 39, 38], [18, 17, 16, 39, 38, 37], [18, 16, 15, 39, 38, 37],
                        [18, 15, 17, 39, 38, 37, 36], [18, 17, 16, 39, 38, 37, 36, 35]]
    expected_last = [3, 2, 1, 4, 3, 2]
    for vis, last in zip(expected_visible, expected_last):
        plan = pol.append_frame(); pol.evict_frames(1, 2)
        ht.step([{"ops": OP_APPEND | OP_EVICT, "sliding_window": 2}], append=True)
        assert ht.append_rows.tolist() == plan.rows(4)
        ids, lens, _ = ht.visible(pol.visible_tokens())
        assert ids == vis and lens[-1] == last
        check_same(ht, pol)


@pytest.mark.parametrize("layout", [LAYOUT_TWO_STREAM, LAYOUT_FRAME_PAGES])
@pytest.mark.parametrize("page_size,n_special", [(None, 5), (4, 5), (16, 5), (3, 7)])
def test_random_scripts_match_oracle(host_lib, layout, page_size, n_special):
    rng = random.Random(hash((layout, page_size)) & 0xffff)
    T = 37
    pol = PagePolicy(T, n_special, page_size, 2, 3, max_total_frames=300, layout=layout)
    ht = HostTables(host_lib, pol, max_total_frames=300)
    for step in range(250):
        r = rng.random()
        kw = {}
        if layout == LAYOUT_FRAME_PAGES:
            kw = rng.choice([{}, {}, {"camera_only": True}, {"cross_frame_special": False}])
        keep = pol._keep_tokens(kw.get("cross_frame_special", True), kw.get("camera_only", False)) \
            if layout == LAYOUT_FRAME_PAGES else 0
        if r < 0.5:      # keyframe, fused into one call
            plan = pol.append_frame(); pol.evict_frames(2, 3, **kw)
            ht.step([{"ops": OP_APPEND | OP_EVICT | OP_PLAN, "sliding_window": 3, "keep_tokens": keep,
                      "expect_kv_tokens": pol.visible_tokens()}], append=True, plan=True)
            assert ht.append_rows.tolist() == plan.rows(pol.page_size)
        elif r < 0.7:    # non-keyframe the reference way: append, attend, roll back
            plan = pol.append_frame()
            ht.step([{"ops": OP_APPEND}], append=True)
            assert ht.append_rows.tolist() == plan.rows(pol.page_size)
            check_same(ht, pol)
            pol.rollback_last_frame()
            ht.step([{"ops": OP_ROLLBACK}])
        elif r < 0.8:    # non-keyframe with a read-only tail: nothing changes, rows get a tail
            n = pol.visible_tokens()
            _, _, rows = ht.visible(n + T, self_tokens=T)
            assert rows[:n] == oracle_rows(pol) and rows[n:] == [-1 - t for t in range(T)]
        elif r < 0.9:    # deferred eviction executed later
            pol.append_frame()
            ht.step([{"ops": OP_APPEND}], append=True)
            pol.execute_deferred_eviction(2, 3, **kw)
            ht.step([{"ops": OP_EVICT, "sliding_window": 3, "keep_tokens": keep}])
        elif r < 0.93:
            pol.reset(); ht.step([{"ops": OP_RESET}])
        else:            # rollback fused with the next keyframe's append
            if pol.frame_count == 0:
                continue
            pol.rollback_last_frame(); pol.append_frame(); pol.evict_frames(2, 3, **kw)
            ht.step([{"ops": OP_ROLLBACK | OP_APPEND | OP_EVICT, "sliding_window": 3, "keep_tokens": keep}], append=True)
        check_same(ht, pol)


def test_two_streams_are_independent_and_offset(host_lib):
    pol0 = PagePolicy(23, 5, 4, 1, 2, max_total_frames=40, layout=LAYOUT_FRAME_PAGES)
    pol1 = PagePolicy(23, 5, 4, 1, 2, max_total_frames=40, layout=LAYOUT_FRAME_PAGES, page_base=pol0.max_num_pages)
    ht = HostTables(host_lib, pol0, n_streams=2, max_total_frames=40)
    for step in range(12):
        kf1 = step % 3 == 0
        p0 = pol0.append_frame(); pol0.evict_frames(1, 2)
        ops = [{"ops": OP_APPEND | OP_EVICT, "sliding_window": 2, "keep_tokens": 5}, {"ops": 0}]
        if kf1:
            p1 = pol1.append_frame(); pol1.evict_frames(1, 2)
            ops[1] = dict(ops[0])
        ht.step(ops, append=True)
        assert ht.append_rows[:23].tolist() == p0.rows(4)
        assert ht.append_rows[23:].tolist() == (p1.rows(4) if kf1 else [-1] * 23)
        check_same(ht, pol0, 0)
        if pol1.frame_count:
            check_same(ht, pol1, 1)


def test_error_word_instead_of_corruption(host_lib):
    pol = PagePolicy(7, 3, None, 1, 2, max_total_frames=1)
    ht = HostTables(host_lib, pol)
    ht.step([{"ops": OP_ROLLBACK}])
    assert ht.hdr()[10] == 16 and ht.hdr()[0] == 0
    ht.step([{"ops": OP_RESET}])
    for _ in range(19):
        ht.step([{"ops": OP_APPEND}], append=True)   # never evicts: pool of 19 pages runs dry
    assert ht.hdr()[10] == 0 or ht.hdr()[10] == 2    # the special pool (17 pages) may run dry first
    before = ht.tables.copy()
    ht.step([{"ops": OP_APPEND}], append=True)
    assert ht.hdr()[10] & 3 and ht.append_rows.tolist() == [-1] * 7
    after = ht.tables.copy(); after[10] = before[10]
    assert (after == before).all()
    # a wrong host count is flagged and the row table stays inside its bounds
    ht.step([{"ops": OP_RESET}]); ht.step([{"ops": OP_APPEND}], append=True)
    _, _, rows = ht.visible(7 + 3)
    assert ht.hdr()[10] == 32 and rows[7:] == [0, 0, 0]


@pytest.mark.parametrize("page_size", [4, 16, 3])
def test_plan_with_the_newest_frame_named_by_the_callers_rows(host_lib, page_size):
    """LBM_OP_PLAN_NEWEST_SELF: the row table of a step that appends, evicts and plans is the
    ordinary one except for the rows of the frame just appended, which name the caller's rows
    (-1 - (q_begin + t)) in the same place; page lists, counts and the table state are the same.
    Two streams, the second with its own q_begin; anchor frames, a sliding window with evictions
    and trajectory-memory tokens behind the frames."""
    T, n_special = 11, 3
    pols = [PagePolicy(T, n_special, page_size, 1, 3, max_total_frames=12, layout=LAYOUT_FRAME_PAGES) for _ in range(2)]
    keep = pols[0]._keep_tokens(True, False)          # evicted frames leave their special tokens behind
    plain = HostTables(host_lib, pols[0], n_streams=2, max_total_frames=12)
    flagged = HostTables(host_lib, pols[0], n_streams=2, max_total_frames=12)
    visible = [0, 0]
    for frame in range(9):
        for b in range(2):
            if b == 1 and frame % 3 == 2:
                continue      # the second stream skips some frames
            pols[b].append_frame(); pols[b].evict_frames(1, 3)
            visible[b] = pols[b].visible_tokens()
            base = {"sliding_window": 3, "keep_tokens": keep, "expect_kv_tokens": visible[b]}
            per = lambda extra: [dict(base, ops=OP_APPEND | OP_EVICT | OP_PLAN | extra) if i == b else {"ops": 0} for i in range(2)]
            plain.step(per(0), append=True, plan=True)
            flagged.step(per(32), append=True, plan=True)
            assert np.array_equal(plain.tables, flagged.tables) and np.array_equal(plain.append_rows, flagged.append_rows)
            assert np.array_equal(plain.ids, flagged.ids) and np.array_equal(plain.lens, flagged.lens)
            lo = b * plain.rows_cap
            want = plain.kv_rows[lo: lo + visible[b]].copy()
            n_frames = int(plain.hdr(b)[1]) + int(plain.hdr(b)[3])          # anchor + window frames
            first = (n_frames - 1) * T
            assert want[first: first + T].tolist() == plain.append_rows[b * T: (b + 1) * T].tolist()   # the newest frame's pool rows
            want[first: first + T] = -1 - (b * T + np.arange(T))
            assert flagged.kv_rows[lo: lo + visible[b]].tolist() == want.tolist()
            assert flagged.hdr(b)[10] == 0
