"""CPU oracle: page allocator and visible-page-table policy of the streaming KV cache.

TEST INFRASTRUCTURE ONLY.  This module is a plain-Python restatement of the reference's
host-side page bookkeeping.  Only tests, the smoke check and the CPU-baseline leg of the
benchmark may import it; the product path never does.

What is restated, and from where (paths relative to the reference checkout):

* pool sizing and initial free lists      lingbot_map/layers/flashinfer_cache.py:130-170
* patch-page allocation (LIFO ``pop()``)   lingbot_map/layers/flashinfer_cache.py:474-512
* special-stream packing                  lingbot_map/layers/flashinfer_cache.py:514-553
* window eviction (``popleft`` + append)   lingbot_map/layers/flashinfer_cache.py:229-266
* rollback of the last append             lingbot_map/layers/flashinfer_cache.py:268-301
* visible table / last page length        lingbot_map/layers/flashinfer_cache.py:438-470
* occupancy snapshot                      lingbot_map/layers/flashinfer_cache.py:303-322
* reset                                   lingbot_map/layers/flashinfer_cache.py:423-432

Two layouts are provided.

``two_stream`` is the reference's design: patch tokens of a frame go to recyclable patch
pages, special tokens of *every* frame are packed into an append-only special stream.  The
reference fixes ``page_size = patches_per_frame`` (one patch page per frame); here the page
size is free, a frame takes ``ceil(patches_per_frame / page_size)`` patch pages, and with
``page_size == patches_per_frame`` every id sequence is the reference's.

``frame_pages`` is the layout the streaming configurations with 16-token pages prescribe:
the whole frame (specials first) is written to ``ceil(tokens_per_frame / page_size)``
consecutive allocations, and a frame leaving the window is *compacted index-only*: its
leading page(s) stay in the table with the valid length cut to the kept special tokens
(the "trajectory memory"), all other pages return to the free list.  Which tokens are kept
follows the dict-cache eviction of the reference's SDPA path
(lingbot_map/layers/attention.py:676-718: all specials, camera only, or none).

Choices the reference does not fix (it never has more than one page per frame):
a frame's pages are popped one at a time (page ``j`` of the frame is the ``j``-th pop);
eviction pushes a frame's pages back in order ``j = 0, 1, ...``; rollback pushes them back
in reverse so that append followed by rollback restores the free list bit for bit.

Parity pins (tests/test_oracle_policy.py): the hand-derived six-frame trace for
tokens_per_frame=7, the reference's own ``_sanity_check`` figures (8/64/3 pages, 600
specials, last page 88), page conservation after every operation of random scripts, and
equality of the visible token *set* with the dict-cache oracle (oracle/sdpa_cache.py).
"""

from __future__ import annotations

import collections
import math
from dataclasses import dataclass
from typing import Deque, List, Optional, Tuple

LAYOUT_TWO_STREAM = "two_stream"
LAYOUT_FRAME_PAGES = "frame_pages"
HEADROOM_FRAMES = 16  # flashinfer_cache.py:132,135 ("+ 16")


@dataclass
class AppendPlan:
    """Where each token of the appended frame lands: ``(page_id, slot)`` per token."""

    page: List[int]
    slot: List[int]

    def rows(self, page_size: int) -> List[int]:
        """Row index of each token's K vector in a ``[pages, 2, page_size, H, D]`` pool
        flattened to ``[pages * 2 * page_size, H, D]`` (the V row is ``page_size`` later)."""
        return [p * 2 * page_size + s for p, s in zip(self.page, self.slot)]


class PagePolicy:
    """One stream's (or one block's) page tables.  Page ids are offset by ``page_base``."""

    def __init__(
        self,
        tokens_per_frame: int,
        num_special_tokens: int = 6,
        page_size: Optional[int] = None,
        scale_frames: int = 8,
        sliding_window: int = 64,
        max_total_frames: int = 2048,
        layout: str = LAYOUT_TWO_STREAM,
        page_base: int = 0,
    ):
        assert layout in (LAYOUT_TWO_STREAM, LAYOUT_FRAME_PAGES)
        self.layout = layout
        self.tokens_per_frame = tokens_per_frame
        self.num_special_tokens = num_special_tokens
        self.patches_per_frame = tokens_per_frame - num_special_tokens
        assert self.patches_per_frame > 0  # flashinfer_cache.py:113
        self.page_size = self.patches_per_frame if page_size is None else page_size
        assert self.page_size > 0
        self.scale_frames = scale_frames
        self.sliding_window = sliding_window
        self.page_base = page_base
        S = self.page_size
        frames_resident = scale_frames + sliding_window + HEADROOM_FRAMES
        if layout == LAYOUT_TWO_STREAM:
            self.pages_per_frame = math.ceil(self.patches_per_frame / S)
            self.max_patch_pages = frames_resident * self.pages_per_frame
            self.max_special_pages = math.ceil(max_total_frames * num_special_tokens / S) + HEADROOM_FRAMES
            self.keep_pages_max = 0
        else:
            self.pages_per_frame = math.ceil(tokens_per_frame / S)
            self.keep_pages_max = math.ceil(num_special_tokens / S)
            self.max_patch_pages = (
                frames_resident * self.pages_per_frame + max_total_frames * self.keep_pages_max
            )
            self.max_special_pages = 0
        self.max_num_pages = self.max_patch_pages + self.max_special_pages
        self._defer_eviction = False
        self.reset()

    # ------------------------------------------------------------------ state
    def reset(self) -> None:
        b = self.page_base
        self.scale_patch_pages: Deque[List[int]] = collections.deque()
        self.live_window_patch_pages: Deque[List[int]] = collections.deque()
        self.free_patch_pages: List[int] = list(range(b, b + self.max_patch_pages))
        self.all_special_pages: List[int] = []
        self.free_special_pages: List[int] = list(
            range(b + self.max_patch_pages, b + self.max_num_pages)
        )
        self.special_token_count = 0
        # frame_pages only: (kept page ids, kept token count) per compacted frame, oldest first
        self.memory_frames: List[Tuple[List[int], int]] = []
        self.frame_count = 0

    # ----------------------------------------------------------------- append
    def append_frame(self) -> AppendPlan:
        S = self.page_size
        n = self.num_special_tokens
        ppf = self.pages_per_frame
        assert len(self.free_patch_pages) >= ppf, "patch page pool exhausted"
        pages = [self.free_patch_pages.pop() for _ in range(ppf)]
        if len(self.scale_patch_pages) < self.scale_frames:
            self.scale_patch_pages.append(pages)
        else:
            self.live_window_patch_pages.append(pages)

        plan = AppendPlan([0] * self.tokens_per_frame, [0] * self.tokens_per_frame)
        if self.layout == LAYOUT_FRAME_PAGES:
            for t in range(self.tokens_per_frame):
                plan.page[t], plan.slot[t] = pages[t // S], t % S
        else:
            for i in range(self.patches_per_frame):
                plan.page[n + i], plan.slot[n + i] = pages[i // S], i % S
            remaining, written = n, 0
            while remaining > 0:
                tail_offset = self.special_token_count % S
                if tail_offset == 0:
                    assert self.free_special_pages, "special page pool exhausted"
                    self.all_special_pages.append(self.free_special_pages.pop())
                tail_page = self.all_special_pages[-1]
                write_n = min(remaining, S - tail_offset)
                for i in range(write_n):
                    plan.page[written + i], plan.slot[written + i] = tail_page, tail_offset + i
                self.special_token_count += write_n
                written += write_n
                remaining -= write_n
        self.frame_count += 1
        return plan

    # ------------------------------------------------------------------ evict
    def _keep_tokens(self, cross_frame_special: bool, camera_only: bool) -> int:
        if not cross_frame_special:
            return 0
        return 1 if camera_only else self.num_special_tokens

    def _evict(self, sliding_window: int, cross_frame_special: bool, camera_only: bool) -> None:
        S = self.page_size
        while len(self.live_window_patch_pages) > sliding_window:
            pages = self.live_window_patch_pages.popleft()
            kept = 0
            if self.layout == LAYOUT_FRAME_PAGES:
                keep = self._keep_tokens(cross_frame_special, camera_only)
                kept = math.ceil(keep / S)
                if keep:
                    self.memory_frames.append((pages[:kept], keep))
                    self.special_token_count += keep
            for p in pages[kept:]:
                self.free_patch_pages.append(p)

    def evict_frames(
        self,
        scale_frames: Optional[int] = None,
        sliding_window: Optional[int] = None,
        cross_frame_special: bool = True,
        include_scale_frames: bool = True,
        camera_only: bool = False,
        num_register_tokens: int = 4,
    ) -> None:
        if self._defer_eviction:  # flashinfer_cache.py:250-251
            return
        w = self.sliding_window if sliding_window is None else sliding_window
        self._evict(w, cross_frame_special, camera_only)

    def execute_deferred_eviction(
        self, scale_frames: Optional[int] = None, sliding_window: Optional[int] = None, **kw
    ) -> None:
        w = self.sliding_window if sliding_window is None else sliding_window
        self._evict(w, kw.get("cross_frame_special", True), kw.get("camera_only", False))

    # --------------------------------------------------------------- rollback
    def rollback_last_frame(self) -> None:
        assert self.frame_count > 0, "cannot rollback, frame_count is 0"
        if self.frame_count > self.scale_frames:
            pages = self.live_window_patch_pages.pop()
        else:
            pages = self.scale_patch_pages.pop()
        for p in reversed(pages):
            self.free_patch_pages.append(p)
        if self.layout == LAYOUT_TWO_STREAM:
            new_count = self.special_token_count - self.num_special_tokens
            assert new_count >= 0, "special_token_count underflow"
            new_num_pages = math.ceil(new_count / self.page_size) if new_count > 0 else 0
            while len(self.all_special_pages) > new_num_pages:
                self.free_special_pages.append(self.all_special_pages.pop())
            self.special_token_count = new_count
        self.frame_count -= 1

    # ---------------------------------------------------------------- queries
    def _frame_page_lens(self) -> List[int]:
        S, ppf = self.page_size, self.pages_per_frame
        per_frame = self.patches_per_frame if self.layout == LAYOUT_TWO_STREAM else self.tokens_per_frame
        return [S] * (ppf - 1) + [per_frame - (ppf - 1) * S]

    def build_visible_page_table(self) -> List[int]:
        """anchor pages, then window pages, then special / memory pages."""
        out: List[int] = []
        for pages in self.scale_patch_pages:
            out += pages
        for pages in self.live_window_patch_pages:
            out += pages
        if self.layout == LAYOUT_TWO_STREAM:
            out += self.all_special_pages
        else:
            for pages, _ in self.memory_frames:
                out += pages
        return out

    def build_visible_page_lens(self) -> List[int]:
        """Valid tokens in each visible page, same order as the page table."""
        S = self.page_size
        lens: List[int] = []
        fl = self._frame_page_lens()
        for _ in range(len(self.scale_patch_pages) + len(self.live_window_patch_pages)):
            lens += fl
        if self.layout == LAYOUT_TWO_STREAM:
            n = len(self.all_special_pages)
            if n:
                tail = self.special_token_count % S
                lens += [S] * (n - 1) + [S if tail == 0 else tail]
        else:
            for pages, keep in self.memory_frames:
                k = len(pages)
                lens += [S] * (k - 1) + [keep - (k - 1) * S]
        return lens

    def compute_last_page_len(self) -> int:
        lens = self.build_visible_page_lens()
        if self.layout == LAYOUT_TWO_STREAM and not self.all_special_pages:
            # flashinfer_cache.py:463-467 (one page per frame there)
            return self._frame_page_lens()[-1]
        return lens[-1]

    def visible_tokens(self) -> int:
        return sum(self.build_visible_page_lens())

    def get_cache_stats(self) -> dict:
        return {
            "frame_count": self.frame_count,
            "scale_pages": sum(len(p) for p in self.scale_patch_pages),
            "live_pages": sum(len(p) for p in self.live_window_patch_pages),
            "free_pages": len(self.free_patch_pages),
            "special_tokens": self.special_token_count,
        }

    def all_pages_accounted(self) -> bool:
        """Conservation: free, anchor, window, special/memory partition the pool exactly."""
        held: List[int] = list(self.free_patch_pages) + list(self.free_special_pages)
        for pages in self.scale_patch_pages:
            held += pages
        for pages in self.live_window_patch_pages:
            held += pages
        held += self.all_special_pages
        for pages, _ in self.memory_frames:
            held += pages
        b = self.page_base
        return sorted(held) == list(range(b, b + self.max_num_pages))


def is_keyframe(frame_index: int, scale_frames: int, keyframe_interval: int) -> bool:
    """Driver rule, lingbot_map/models/gct_stream.py:450 (frames before ``scale_frames``
    are the anchor pass and always cached)."""
    if frame_index < scale_frames:
        return True
    return keyframe_interval <= 1 or (frame_index - scale_frames) % keyframe_interval == 0
