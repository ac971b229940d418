"""Paged KV-cache manager backed by the gfx950 HIP library.

Drop-in for the reference's ``FlashInferKVCacheManager``
(lingbot_map/layers/flashinfer_cache.py:55-560): same constructor arguments, methods,
attributes and exception types, so the reference's global block
(lingbot_map/layers/block.py:245-285) can drive it unchanged.  What differs is where the
work happens: page tables live on the device and are updated by one index kernel per
operation, the append is one scatter kernel, attention is the MFMA flash kernel.  The host
keeps only *counts* (how many frames, free pages, special tokens), which are a
deterministic function of the call sequence; they back the reference's assertions and
``get_cache_stats`` without ever synchronising with the device.

Extensions beyond the reference signature (all keyword-only, defaults = reference):

``page_size``        tokens per page (reference: patches per frame, one page per frame)
``layout``           ``"two_stream"`` (reference) or ``"frame_pages"`` (whole frame in
                     pages; eviction keeps the leading special tokens index-only)
``num_streams``      independent streams batched in every call (k, v, q are the streams'
                     frames concatenated on the token axis)
``per_block_tables`` one table set per block instead of one shared by all blocks
``device_token_counts`` the attention kernels read each stream's visible-token count from the
                     device tables instead of the launch arguments, so that a frame's launches
                     stay identical while the trajectory memory grows (HIP-graph replay)

With shared tables block 0 leads, as the reference's ``plan()`` at ``block_idx == 0`` does
(flashinfer_cache.py:385-414): table operations run when ``block_idx == 0`` and the other
blocks reuse block 0's latest append plan and attention plan.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Dict, List, Optional, Sequence

import torch
from torch import Tensor

from . import _native as N

HEADROOM_FRAMES = 16  # flashinfer_cache.py:132,135


def _ceil_div(a: int, b: int) -> int:
    return -(-a // b)


class _StreamCounts:
    """Host mirror of one stream's header counts (never page ids)."""

    __slots__ = ("frame_count", "n_anchor", "win_count", "n_free_patch", "n_free_special",
                 "n_special_pages", "special_tokens", "n_memory", "n_memory_pages")

    def __init__(self, patch_pages: int, special_pages: int):
        self.frame_count = self.n_anchor = self.win_count = 0
        self.n_free_patch, self.n_free_special = patch_pages, special_pages
        self.n_special_pages = self.special_tokens = self.n_memory = self.n_memory_pages = 0


class HipPagedKVCacheManager:
    def __init__(
        self,
        num_blocks: int,
        max_num_frames: int,
        tokens_per_frame: int,
        num_heads: int,
        head_dim: int,
        dtype: torch.dtype,
        device: torch.device,
        num_special_tokens: int = 6,
        scale_frames: int = 8,
        sliding_window: int = 64,
        max_total_frames: int = 2048,
        force_fp32: bool = False,
        fa3: bool = False,
        *,
        page_size: Optional[int] = None,
        layout: str = "two_stream",
        num_streams: int = 1,
        per_block_tables: bool = False,
        device_token_counts: bool = False,
    ):
        device = torch.device(device)
        if device.type != "cuda":
            raise RuntimeError("HipPagedKVCacheManager needs a ROCm device; there is no CPU path")
        if layout not in ("two_stream", "frame_pages"):
            raise ValueError(f"unknown layout {layout!r}")
        if not 1 <= num_streams <= N.MAX_STREAMS:
            raise ValueError(f"num_streams must be in [1, {N.MAX_STREAMS}]")
        self.num_blocks = num_blocks
        self.max_num_frames = max_num_frames
        self.num_special_tokens = num_special_tokens
        self.patches_per_frame = tokens_per_frame - num_special_tokens
        assert self.patches_per_frame > 0, (
            f"tokens_per_frame={tokens_per_frame} <= num_special_tokens={num_special_tokens}")
        if page_size is None:
            p = self.patches_per_frame
            page_size = 1 << (p - 1).bit_length() if fa3 else p  # flashinfer_cache.py:100-106
        assert page_size > 0
        self.page_size = page_size
        self.scale_frames = scale_frames
        # one window for all streams, or one per stream (ragged batch)
        if isinstance(sliding_window, (list, tuple)):
            assert len(sliding_window) == num_streams, "one sliding_window per stream"
            self._windows = [int(w) for w in sliding_window]
            self._ragged_windows = True
            sliding_window = max(self._windows)
        else:
            self._windows = [int(sliding_window)] * num_streams
            self._ragged_windows = False
        self.sliding_window = sliding_window
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.tokens_per_frame = tokens_per_frame
        self.layout = layout
        self.num_streams = num_streams
        self.per_block_tables = per_block_tables
        self.device_token_counts = bool(device_token_counts)
        self.force_fp32 = force_fp32
        if force_fp32:  # flashinfer_cache.py:121-127
            self.dtype = torch.float32
        else:
            self.dtype = torch.bfloat16 if dtype == torch.float32 else dtype
        if self.dtype not in (torch.bfloat16, torch.float32):
            raise RuntimeError(f"unsupported cache dtype {self.dtype}")
        self.device = device

        S = page_size
        two = layout == "two_stream"
        resident = scale_frames + sliding_window + HEADROOM_FRAMES
        if two:
            self._tpf = self.patches_per_frame
            self.pages_per_frame = _ceil_div(self._tpf, S)
            self.max_patch_pages = resident * self.pages_per_frame
            self.max_special_pages = _ceil_div(max_total_frames * num_special_tokens, S) + HEADROOM_FRAMES
            self._keep_pages_max, memory_frames = 0, 0
        else:
            self._tpf = tokens_per_frame
            self.pages_per_frame = _ceil_div(self._tpf, S)
            self._keep_pages_max = _ceil_div(num_special_tokens, S)
            self.max_patch_pages = resident * self.pages_per_frame + max_total_frames * self._keep_pages_max
            self.max_special_pages, memory_frames = 0, max_total_frames
        self.max_num_pages = self.max_patch_pages + self.max_special_pages
        self._ring_frames = self.max_patch_pages // self.pages_per_frame
        self._geom = N.CacheGeom(
            N.LAYOUT_TWO_STREAM if two else N.LAYOUT_FRAME_PAGES, tokens_per_frame, num_special_tokens, S,
            scale_frames, self.max_patch_pages, self.max_special_pages, memory_frames, self.max_num_pages)
        words = N.lib.lbm_tables_words(C.byref(self._geom))
        if words <= 0:
            raise ValueError("invalid cache geometry")
        self._table_words = int(words)

        # ── device memory: pools, tables, plans ──────────────────────────────
        self.kv_caches: List[Tensor] = [
            torch.zeros(num_streams * self.max_num_pages, 2, S, num_heads, head_dim, dtype=self.dtype, device=device)
            for _ in range(num_blocks)
        ]
        self._n_sets = num_blocks if per_block_tables else 1
        self._tables = torch.zeros(self._n_sets, num_streams, self._table_words, dtype=torch.int32, device=device)
        T = tokens_per_frame
        self._rows_cap = (self._ring_frames + scale_frames) * self._tpf + T + (
            self.max_special_pages * S if two else memory_frames * num_special_tokens)
        self._pages_cap = (self._ring_frames + scale_frames) * self.pages_per_frame + (
            self.max_special_pages if two else memory_frames * self._keep_pages_max)
        self._append_rows = torch.full((self._n_sets, num_streams * T), -1, dtype=torch.int32, device=device)
        self._kv_rows = torch.zeros(self._n_sets, num_streams * self._rows_cap, dtype=torch.int32, device=device)
        self._page_ids = torch.zeros(num_streams * self._pages_cap, dtype=torch.int32, device=device)
        self._page_lens = torch.zeros(num_streams * self._pages_cap, dtype=torch.int32, device=device)
        self.workspace_buffer = torch.empty(0, dtype=torch.uint8, device=device)

        # ── host state ───────────────────────────────────────────────────────
        self.frame_count: List[int] = [0] * num_blocks
        self._defer_eviction: bool = False
        self._skip_append: bool = False
        self._counts = [[_StreamCounts(self.max_patch_pages, self.max_special_pages) for _ in range(num_streams)]
                        for _ in range(self._n_sets)]
        # streams taking part in the current step (all by default)
        self._active: List[bool] = [True] * num_streams
        # visible-token counts and self-tail flags of the latest plan of each table set
        self._plan_tokens = [[0] * num_streams for _ in range(self._n_sets)]
        self._plan_valid = [False] * self._n_sets
        # append rows of frames block 0 wrote while other blocks were still behind (anchor pass)
        self._rows_log: Dict[int, Tensor] = {}
        #: step(): the attention call stores the new frame itself (lbm_attn_run_append), reading it
        #: from the caller's tensors meanwhile - no append launch in front of the attention
        self.fuse_append = True
        self._newest_self = [False] * self._n_sets   # the set's row table names the newest frame by the caller's rows
        self._n_appends: List[int] = [0] * num_blocks    # appends ever made per block (rollbacks do not count down)
        self.reset()

    # =========================================================================
    # helpers
    # =========================================================================
    def _stream_handle(self):
        return N.stream_ptr(self.device)

    def _set(self, block_idx: int) -> int:
        return block_idx if self.per_block_tables else 0

    def _leads(self, block_idx: int) -> bool:
        return self.per_block_tables or block_idx == 0

    def _ops(self, per_stream: Sequence[dict]):
        arr = (N.StepOp * self.num_streams)()
        for b, d in enumerate(per_stream):
            arr[b].q_begin = b * self.tokens_per_frame
            arr[b].kv_row_begin = b * self._rows_cap
            arr[b].page_out_begin = b * self._pages_cap
            for k, v in d.items():
                setattr(arr[b], k, v)
        return arr

    def _tables_step(self, ts: int, ops, append_rows=False, kv_rows=False, pages=False) -> None:
        N.check(N.lib.lbm_tables_step(
            C.c_void_p(self._tables[ts].data_ptr()), C.byref(self._geom), self.num_streams, ops,
            C.c_void_p(self._append_rows[ts].data_ptr()) if append_rows else None,
            C.c_void_p(self._kv_rows[ts].data_ptr()) if kv_rows else None,
            C.c_void_p(self._page_ids.data_ptr()) if pages else None,
            C.c_void_p(self._page_lens.data_ptr()) if pages else None,
            self._stream_handle()))

    def _expect(self, n: int) -> int:
        """PLAN's token argument: the host's count, or - with device-side counts - minus the
        capacity of the stream's row table."""
        return -self._rows_cap if self.device_token_counts else n

    def _visible_tokens(self, c: _StreamCounts) -> int:
        return (c.n_anchor + c.win_count) * self._tpf + c.special_tokens

    def _window_of(self, stream: int, requested: int) -> int:
        """Window of one stream: the caller's value (as in the reference), or the stream's own
        window when the manager was built with one window per stream."""
        return self._windows[stream] if self._ragged_windows else requested

    def _keep_tokens(self, cross_frame_special: bool, camera_only: bool) -> int:
        # lingbot_map/layers/attention.py:690-696
        if self.layout == "two_stream" or not cross_frame_special:
            return 0
        return 1 if camera_only else self.num_special_tokens

    def set_active_streams(self, active: Optional[Sequence[bool]]) -> None:
        """Streams that take part in the following calls (None = all).  A stream that is
        not active keeps its tables, gets no K/V written and no attention output."""
        self._active = [True] * self.num_streams if active is None else [bool(a) for a in active]
        assert len(self._active) == self.num_streams

    # ----- host mirror transitions (same arithmetic as the device phases) -----
    def _mirror_append(self, c: _StreamCounts, block_idx: int) -> None:
        ppf, S, n = self.pages_per_frame, self.page_size, self.num_special_tokens
        assert c.n_free_patch >= ppf, (
            f"block {block_idx}: patch page pool exhausted — scale={c.n_anchor * ppf}, "
            f"window={c.win_count * ppf}, free={c.n_free_patch}")
        if self.layout == "two_stream":
            new_sp = _ceil_div(c.special_tokens + n, S) - c.n_special_pages
            assert new_sp <= c.n_free_special, (
                f"block {block_idx}: special page pool exhausted at special_token_count={c.special_tokens}. "
                f"Increase max_total_frames.")
            c.n_free_special -= new_sp
            c.n_special_pages += new_sp
            c.special_tokens += n
        if c.n_anchor < self.scale_frames:
            c.n_anchor += 1
        else:
            c.win_count += 1
        c.n_free_patch -= ppf
        c.frame_count += 1

    def _mirror_evict(self, c: _StreamCounts, window: int, keep: int, block_idx: int) -> None:
        n_ev = c.win_count - window
        if n_ev <= 0:
            return
        kp = _ceil_div(keep, self.page_size) if keep else 0
        if keep:
            assert c.n_memory + n_ev <= self._geom.memory_frames, (
                f"block {block_idx}: trajectory memory full ({c.n_memory} frames). Increase max_total_frames.")
            c.n_memory += n_ev
            c.n_memory_pages += n_ev * kp
            c.special_tokens += n_ev * keep
        c.win_count -= n_ev
        c.n_free_patch += n_ev * (self.pages_per_frame - kp)

    def _mirror_rollback(self, c: _StreamCounts, block_idx: int) -> None:
        assert c.frame_count > 0, f"block {block_idx}: cannot rollback, frame_count is 0"
        if c.frame_count > self.scale_frames:
            assert c.win_count > 0, f"block {block_idx}: cannot rollback, window is empty"
            c.win_count -= 1
        else:
            c.n_anchor -= 1
        c.n_free_patch += self.pages_per_frame
        if self.layout == "two_stream":
            n = self.num_special_tokens
            new_count = c.special_tokens - n
            assert new_count >= 0, (
                f"block {block_idx}: special_token_count underflow ({c.special_tokens} - {n})")
            new_pages = _ceil_div(new_count, self.page_size) if new_count > 0 else 0
            c.n_free_special += c.n_special_pages - new_pages
            c.n_special_pages = new_pages
            c.special_tokens = new_count
        c.frame_count -= 1

    # =========================================================================
    # Public API (flashinfer_cache.py:202-560)
    # =========================================================================
    def _check_frame(self, name: str, x: Tensor) -> Tensor:
        rows = self.num_streams * self.tokens_per_frame
        assert x.dim() == 3 and x.shape[0] == rows and x.shape[1] == self.num_heads and x.shape[2] == self.head_dim, (
            f"{name}: expected [{rows}, {self.num_heads}, {self.head_dim}], got {tuple(x.shape)}")
        if x.dtype not in (torch.bfloat16, torch.float32):
            x = x.to(self.dtype)
        return x.contiguous()

    def append_frame(self, block_idx: int, k: Tensor, v: Tensor) -> None:
        k, v = self._check_frame("k", k), self._check_frame("v", v)
        if v.dtype != k.dtype:
            v = v.to(k.dtype)
        ts = self._set(block_idx)
        rows = self._append_rows[ts]
        if self._leads(block_idx):
            if self._others_behind():
                # the anchor pass appends several frames block by block (attention.py:497-511):
                # the other blocks still have to write the frame appended last, keep its rows
                self._rows_log[self._n_appends[0] - 1] = rows.clone()
            for b in range(self.num_streams):
                if self._active[b]:
                    self._mirror_append(self._counts[ts][b], block_idx)
            ops = self._ops([{"ops": N.OP_APPEND if self._active[b] else 0} for b in range(self.num_streams)])
            self._tables_step(ts, ops, append_rows=True)
            self._plan_valid[ts] = False
        else:
            n, lead = self._n_appends[block_idx], self._n_appends[0]
            if n >= lead:
                raise RuntimeError(f"block {block_idx} makes its append number {n} before block 0 has: with shared "
                                   "page tables block 0 goes first (or build the manager with per_block_tables=True)")
            if n < lead - 1:
                rows = self._rows_log.get(n)
                if rows is None:
                    raise RuntimeError(f"block {block_idx} has made {n} appends, block 0 {lead}, and the rows of "
                                       "that frame are no longer known (block 0 evicted or rolled back in between); blocks that "
                                       "run that far apart need per_block_tables=True")
        self._scatter(block_idx, rows, k, v)
        self.frame_count[block_idx] += 1
        self._n_appends[block_idx] += 1
        if self._rows_log and not self._leads(block_idx):
            done = min(self._n_appends[1:])
            for f in [f for f in self._rows_log if f < done]:
                del self._rows_log[f]

    def _others_behind(self) -> bool:
        """Shared page tables only: some block has not yet written the frame block 0 appended last."""
        return (not self.per_block_tables and self.num_blocks > 1
                and min(self._n_appends[1:]) < self._n_appends[0])

    def _in_step(self, block_idx: int, what: str) -> None:
        """Shared page tables describe the frames block 0 has appended; another block may use
        them only once it has written the same frames."""
        if not self._leads(block_idx) and self._n_appends[block_idx] != self._n_appends[0]:
            raise RuntimeError(f"{what}: block {block_idx} has made {self._n_appends[block_idx]} appends, block 0 "
                               f"{self._n_appends[0]}; with shared page tables every block handles a frame before "
                               "block 0 moves on (only the anchor pass may append block by block)")

    def _scatter(self, block_idx: int, rows: Tensor, k: Tensor, v: Tensor) -> None:
        N.check(N.lib.lbm_kv_append(
            C.c_void_p(k.data_ptr()), C.c_void_p(v.data_ptr()),
            N.DTYPE_BF16 if k.dtype == torch.bfloat16 else N.DTYPE_F32,
            C.c_void_p(self.kv_caches[block_idx].data_ptr()),
            N.DTYPE_BF16 if self.dtype == torch.bfloat16 else N.DTYPE_F32,
            C.c_void_p(rows.data_ptr()), k.shape[0], self.num_heads, self.head_dim,
            self.page_size, self._stream_handle()))

    def evict_frames(self, block_idx: int, scale_frames: int, sliding_window: int,
                     cross_frame_special: bool = True, include_scale_frames: bool = True,
                     camera_only: bool = False, num_register_tokens: int = 4) -> None:
        if self._defer_eviction:  # flashinfer_cache.py:250-251
            return
        self._evict(block_idx, sliding_window, cross_frame_special, camera_only)

    def execute_deferred_eviction(self, block_idx: int, scale_frames: int, sliding_window: int, **kwargs) -> None:
        self._evict(block_idx, sliding_window, kwargs.get("cross_frame_special", True), kwargs.get("camera_only", False))

    def _evict(self, block_idx: int, sliding_window: int, cross_frame_special: bool, camera_only: bool) -> None:
        if not self._leads(block_idx):
            return
        ts = self._set(block_idx)
        keep = self._keep_tokens(cross_frame_special, camera_only)
        todo = False
        for b in range(self.num_streams):
            c = self._counts[ts][b]
            w = self._window_of(b, sliding_window)
            if self._active[b] and c.win_count > w:
                self._mirror_evict(c, w, keep, block_idx)
                todo = True
        if not todo:
            return
        self._rows_log.clear()   # evicted pages may be handed out again: a block still behind raises
        ops = self._ops([{"ops": N.OP_EVICT if self._active[b] else 0, "sliding_window": self._window_of(b, sliding_window),
                          "keep_tokens": keep} for b in range(self.num_streams)])
        self._tables_step(ts, ops)
        self._plan_valid[ts] = False

    def rollback_last_frame(self, block_idx: int) -> None:
        assert self.frame_count[block_idx] > 0, f"block {block_idx}: cannot rollback, frame_count is 0"
        if self._leads(block_idx):
            ts = self._set(block_idx)
            self._rows_log.clear()
            for b in range(self.num_streams):
                if self._active[b]:
                    self._mirror_rollback(self._counts[ts][b], block_idx)
            ops = self._ops([{"ops": N.OP_ROLLBACK if self._active[b] else 0} for b in range(self.num_streams)])
            self._tables_step(ts, ops)
            # the attention plan of the rolled-back frame stays valid for the following blocks
        self.frame_count[block_idx] -= 1

    def get_cache_stats(self, block_idx: int = 0, stream: int = 0) -> dict:
        c = self._counts[self._set(block_idx)][stream]
        return {
            "frame_count": int(self.frame_count[block_idx]),
            "scale_pages": c.n_anchor * self.pages_per_frame,
            "live_pages": c.win_count * self.pages_per_frame,
            "free_pages": c.n_free_patch,
            "special_tokens": c.special_tokens,
        }

    def _plan(self, ts: int, self_tail: Sequence[bool], pages: bool = False) -> None:
        per = []
        for b in range(self.num_streams):
            c = self._counts[ts][b]
            tail = self.tokens_per_frame if self_tail[b] else 0
            n = self._visible_tokens(c) + tail if self._active[b] else 0
            self._plan_tokens[ts][b] = n
            per.append({"ops": N.OP_PLAN if self._active[b] else 0, "self_tokens": tail,
                        "expect_kv_tokens": self._expect(n)})
        self._tables_step(ts, self._ops(per), kv_rows=True, pages=pages)
        self._plan_valid[ts] = True
        self._newest_self[ts] = False

    def compute_attention(self, block_idx: int, q: Tensor, self_k: Optional[Tensor] = None,
                          self_v: Optional[Tensor] = None) -> Tensor:
        """softmax(q K^T / sqrt(D)) V over every visible cached token.

        ``self_k``/``self_v`` (optional, same shape as ``q``) are attended to as well without
        being stored: the read-only path of a non-keyframe (block.py:256-263 does the same
        by appending, attending and rolling back)."""
        has_tail = self_k is not None
        if self.frame_count[block_idx] == 0 and not has_tail:
            return torch.zeros_like(q)  # flashinfer_cache.py:368-370
        ts = self._set(block_idx)
        self._in_step(block_idx, "compute_attention")
        if self._leads(block_idx) or not self._plan_valid[ts]:
            self._plan(ts, [has_tail and self._active[b] for b in range(self.num_streams)])
        return self._attend_planned(block_idx, q, self_k, self_v)

    def step(self, block_idx: int, q: Tensor, k: Tensor, v: Tensor, keyframe: Optional[Sequence[bool]] = None,
             cross_frame_special: bool = True, camera_only: bool = False) -> Tensor:
        """One frame of every stream through one block: keyframes append, evict and attend;
        the others attend to the cache plus their own K/V and leave it untouched.  On the
        leading block all table work (allocate, evict, visible rows) is one launch."""
        k, v = self._check_frame("k", k), self._check_frame("v", v)
        if v.dtype != k.dtype:
            v = v.to(k.dtype)
        want = self.fuse_append and self.layout == "frame_pages" and not self.device_token_counts
        ts, keyframe, tail = self._step_tables(block_idx, keyframe, cross_frame_special, camera_only, newest_self=want)
        if self._newest_self[ts]:
            # the row table names the keyframes' new rows by k and v themselves: attend, then store
            # them, in one call
            self.frame_count[block_idx] += 1
            self._n_appends[block_idx] += 1
            return self._attend_planned(block_idx, q, k, v, append_rows=self._append_rows[ts])
        if any(keyframe):
            self._scatter(block_idx, self._append_rows[ts], k, v)
            self.frame_count[block_idx] += 1
            self._n_appends[block_idx] += 1
        return self._attend_planned(block_idx, q, k if any(tail) else None, v if any(tail) else None)

    def step_qkv(self, block_idx: int, qkv: Optional[Tensor], q_norm=None, k_norm=None, rope_cs: Optional[Tensor] = None,
                 norm_eps: float = 1e-5, keyframe: Optional[Sequence[bool]] = None,
                 cross_frame_special: bool = True, camera_only: bool = False, proj=None) -> Tensor:
        """`step` fed with the output of the qkv projection instead of finished q, k, v: one
        kernel applies the per-head LayerNorm of q and k, the rotary embedding, lays q out as
        [token, head, dim] and writes k and v straight into the page pool (attention.py:402-426
        plus append_frame).  ``qkv``: [streams * tokens_per_frame, 3 * heads * head_dim];
        ``q_norm`` / ``k_norm``: (weight, bias) float32 tensors of [head_dim] or None;
        ``rope_cs``: float32 [streams * tokens_per_frame, head_dim / 2, 2] holding (cos, sin),
        i.e. ``torch.view_as_real`` of the reference's complex ``freqs``, or None.

        ``proj = (x, weight, bias)`` instead of ``qkv`` (then None): the projection itself runs in
        the same kernel (``x`` [rows, K] bf16, ``weight`` [3 * heads * head_dim, K] bf16, ``bias``
        float32 or None; bf16 cache, head_dim 64) and its output never goes to memory; the results
        are bit-identical to projecting first."""
        rows, H, D = self.num_streams * self.tokens_per_frame, self.num_heads, self.head_dim
        if proj is None:
            assert qkv.shape[0] == rows and qkv.numel() == rows * 3 * H * D, (
                f"qkv: expected [{rows}, {3 * H * D}], got {tuple(qkv.shape)}")
            if qkv.dtype not in (torch.bfloat16, torch.float32):
                qkv = qkv.to(self.dtype)
            qkv = qkv.contiguous()
        else:
            px, pw, pb = proj[:3]
            row_norm = proj[3] if len(proj) > 3 else None   # lbm_row_norm: norm1 folded into the projection
            assert qkv is None and self.dtype == torch.bfloat16 and D == 64, "proj: bf16 cache with head_dim 64"
            assert px.dtype == pw.dtype == torch.bfloat16 and px.is_contiguous() and pw.is_contiguous()
            assert px.shape[0] == rows and pw.shape == (3 * H * D, px.shape[1]) and px.shape[1] % 128 == 0, (
                f"proj: x [{rows}, K] and weight [{3 * H * D}, K] with K a multiple of 128, got {tuple(px.shape)}, {tuple(pw.shape)}")
            assert pb is None or (pb.dtype == torch.float32 and pb.numel() == 3 * H * D)
        assert (q_norm is None) == (k_norm is None), "q_norm and k_norm go together"
        ts, keyframe, tail = self._step_tables(block_idx, keyframe, cross_frame_special, camera_only)
        q = torch.empty(rows, H, D, dtype=self.dtype, device=self.device)
        k = torch.empty_like(q) if any(tail) else None
        v = torch.empty_like(q) if any(tail) else None
        # float32 copies of the LayerNorm parameters, kept alive until the launch is queued
        norm = [self._as_f32(t, D) for t in (tuple(q_norm) + tuple(k_norm))] if q_norm is not None else [None] * 4
        norm_ptr = [None if t is None else C.c_void_p(t.data_ptr()) for t in norm]
        if rope_cs is not None:
            assert rope_cs.dtype == torch.float32 and rope_cs.numel() == rows * D, (
                f"rope_cs: expected float32 [{rows}, {D // 2}, 2], got {rope_cs.dtype} {tuple(rope_cs.shape)}")
            rope_cs = rope_cs.contiguous()
        dt = lambda d: N.DTYPE_BF16 if d == torch.bfloat16 else N.DTYPE_F32
        vp = lambda t: None if t is None else C.c_void_p(t.data_ptr())
        rope_ptr = vp(rope_cs)
        append_ptr = vp(self._append_rows[ts]) if any(keyframe) else None
        # q leaves the producer multiplied by the softmax scale and log2(e) - one rounding for the
        # row instead of the producer's and then the attention kernel's - and the attention call
        # below is told so (sm_scale = 0)
        q_scale = N.q_scale_log2(1.0 / math.sqrt(D))
        if proj is None:
            N.check(N.lib.lbm_qkv_prepare(
                vp(qkv), dt(qkv.dtype), norm_ptr[0], norm_ptr[1], norm_ptr[2], norm_ptr[3], float(norm_eps), q_scale,
                rope_ptr, N.ROPE_INTERLEAVED, vp(q), vp(k), vp(v), dt(self.dtype),
                vp(self.kv_caches[block_idx]), append_ptr, rows, H, D, self.page_size, self._stream_handle()))
        else:
            N.check(N.lib.lbm_qkv_linear_prepare_norm(
                vp(px), row_norm, vp(pw), vp(pb), rows, px.shape[1], norm_ptr[0], norm_ptr[1], norm_ptr[2], norm_ptr[3],
                float(norm_eps), q_scale, rope_ptr, N.ROPE_INTERLEAVED, vp(q), vp(k), vp(v),
                vp(self.kv_caches[block_idx]), append_ptr, H, D, self.page_size, self._stream_handle()))
        if any(keyframe):
            self.frame_count[block_idx] += 1
            self._n_appends[block_idx] += 1
        return self._attend_planned(block_idx, q, k, v, q_prescaled=True)

    def _as_f32(self, t: Tensor, n: int) -> Tensor:
        assert t.numel() == n, f"expected {n} LayerNorm parameters, got {tuple(t.shape)}"
        return t if (t.dtype == torch.float32 and t.is_contiguous() and t.device == self.device) else \
            t.detach().to(device=self.device, dtype=torch.float32).contiguous()

    def steady_state(self, cross_frame_special: bool = True, camera_only: bool = False) -> bool:
        """True when one more keyframe step of every active stream would launch exactly what
        the last one launched - the condition under which a captured HIP graph of a frame may be
        replayed (page ids live on the device and keep evolving across replays).  Anchor and
        window must be full.  With host-side token counts the visible token count must not change
        either, i.e. evicted frames must leave no memory tokens; with ``device_token_counts`` the
        kernels read the count on the device and the trajectory memory may grow."""
        if self._skip_append or self._defer_eviction or not any(self._active):
            return False
        keep = self._keep_tokens(cross_frame_special, camera_only)
        for ts in range(self._n_sets):
            for b in range(self.num_streams):
                if not self._active[b]:
                    continue
                c = self._counts[ts][b]
                probe = _StreamCounts(0, 0)
                for f in _StreamCounts.__slots__:
                    setattr(probe, f, getattr(c, f))
                before = self._visible_tokens(c)
                self._mirror_append(probe, 0)
                self._mirror_evict(probe, self._windows[b], keep, 0)
                grows = ("frame_count", "n_memory", "n_memory_pages", "special_tokens", "n_free_patch") \
                    if self.device_token_counts and self.layout == "frame_pages" else ("frame_count",)
                same = all(getattr(probe, f) == getattr(c, f) for f in _StreamCounts.__slots__ if f not in grows)
                if not same or not self._plan_valid[ts]:
                    return False
                if not self.device_token_counts and self._visible_tokens(probe) != before:
                    return False
        return True

    def note_replayed_frames(self, n: int = 1, cross_frame_special: bool = True, camera_only: bool = False) -> None:
        """Book-keeping after replaying a captured steady-state keyframe ``n`` times (``n = -1``
        takes back the host side of a frame that was only captured, not executed): the device
        tables advanced, the host's mirror follows."""
        keep = self._keep_tokens(cross_frame_special, camera_only)
        for i in range(self.num_blocks):
            self.frame_count[i] += n
            self._n_appends[i] += n
        for ts in range(self._n_sets):
            for b in range(self.num_streams):
                if not self._active[b]:
                    continue
                c = self._counts[ts][b]
                if n < 0 or keep == 0:
                    c.frame_count += n
                    if n < 0 and keep:   # undo the memory growth of the captured frame
                        kp = _ceil_div(keep, self.page_size)
                        c.n_memory += n
                        c.n_memory_pages += n * kp
                        c.special_tokens += n * keep
                        c.n_free_patch -= n * kp
                    self._plan_tokens[ts][b] = self._visible_tokens(c)
                    continue
                for _ in range(n):
                    self._mirror_append(c, 0)
                    self._mirror_evict(c, self._windows[b], keep, 0)
                self._plan_tokens[ts][b] = self._visible_tokens(c)

    def _step_tables(self, block_idx: int, keyframe: Optional[Sequence[bool]], cross_frame_special: bool,
                     camera_only: bool, newest_self: bool = False):
        """Table work of one streamed frame (allocate, evict, visible rows; one launch on the
        leading block).  Returns the table set and the per-stream keyframe / read-only flags.
        ``newest_self`` (leading block): the row table names the rows a keyframe appends by the
        caller's own K/V rows; every block of the frame then attends and appends with
        ``lbm_attn_run_append`` (``step`` does), which ``_newest_self`` remembers."""
        if keyframe is None:
            keyframe = [not self._skip_append] * self.num_streams
        keyframe = [bool(x) and self._active[b] for b, x in enumerate(keyframe)]
        tail = [self._active[b] and not keyframe[b] for b in range(self.num_streams)]
        ts = self._set(block_idx)
        if self._leads(block_idx):
            if self._others_behind():
                raise RuntimeError(f"step: block 0 starts a frame while another block has made "
                                   f"{min(self._n_appends[1:])} of its {self._n_appends[0]} appends")
            keep = self._keep_tokens(cross_frame_special, camera_only)
            per = []
            for b in range(self.num_streams):
                c = self._counts[ts][b]
                ops, n = 0, 0
                if keyframe[b]:
                    self._mirror_append(c, block_idx)
                    ops = N.OP_APPEND | N.OP_PLAN | (N.OP_PLAN_NEWEST_SELF if newest_self else 0)
                    if not self._defer_eviction:
                        self._mirror_evict(c, self._windows[b], keep, block_idx)
                        ops |= N.OP_EVICT
                    n = self._visible_tokens(c)
                elif tail[b]:
                    ops = N.OP_PLAN
                    n = self._visible_tokens(c) + self.tokens_per_frame
                self._plan_tokens[ts][b] = n
                per.append({"ops": ops, "sliding_window": self._windows[b], "keep_tokens": keep,
                            "self_tokens": self.tokens_per_frame if tail[b] else 0,
                            "expect_kv_tokens": self._expect(n)})
            self._tables_step(ts, self._ops(per), append_rows=True, kv_rows=True)
            self._plan_valid[ts] = True
            self._newest_self[ts] = bool(newest_self and any(keyframe))
        elif self._n_appends[block_idx] + (1 if any(keyframe) else 0) != self._n_appends[0]:
            raise RuntimeError(f"step: block {block_idx} has made {self._n_appends[block_idx]} appends, block 0 "
                               f"{self._n_appends[0]}: with shared page tables every block takes the frame block 0 took")
        return ts, keyframe, tail

    def _attend_planned(self, block_idx: int, q: Tensor, self_k: Optional[Tensor], self_v: Optional[Tensor],
                        q_prescaled: bool = False, append_rows: Optional[Tensor] = None) -> Tensor:
        """``q_prescaled``: q already carries 1 / sqrt(D) and log2(e) (``step_qkv``'s producer).
        ``append_rows``: ``self_k`` / ``self_v`` are also stored, row t in pool row
        ``append_rows[t]``, once the attention has read the pool (``lbm_attn_run_append``)."""
        ts = self._set(block_idx)
        if self._newest_self[ts] and append_rows is None:
            raise RuntimeError("this frame's row table names its newest frame by the caller's K/V rows (step() led "
                               "the frame): every block of the frame takes it through step()")
        rows = self.num_streams * self.tokens_per_frame
        assert q.dim() == 3 and tuple(q.shape) == (rows, self.num_heads, self.head_dim), (
            f"q: expected [{rows}, {self.num_heads}, {self.head_dim}], got {tuple(q.shape)}")
        qc = q.to(self.dtype).contiguous()
        out = torch.empty_like(qc)
        has_tail = self_k is not None
        if has_tail:
            self_k = self_k.to(self.dtype).contiguous()
            self_v = self_v.to(self.dtype).contiguous()
        streams = (N.AttnStream * self.num_streams)()
        n, T = 0, self.tokens_per_frame
        for b in range(self.num_streams):
            kv = self._plan_tokens[ts][b]
            if kv > 0:
                streams[n] = N.AttnStream(b * T, T, b * self._rows_cap, kv, b * self._table_words)
                n += 1
        if n < self.num_streams:
            out.zero_()
        if n == 0:
            if append_rows is not None:
                self._scatter(block_idx, append_rows, self_k, self_v)
            return out
        need = N.lib.lbm_attn_workspace_bytes(streams, n, self.num_heads, self.head_dim)
        if need > self.workspace_buffer.numel():
            self.workspace_buffer = torch.empty(int(need * 1.25) + 256, dtype=torch.uint8, device=self.device)
        common = (streams, n, self.num_heads, self.head_dim, self.page_size,
                  N.DTYPE_BF16 if self.dtype == torch.bfloat16 else N.DTYPE_F32,
                  0.0 if q_prescaled else 1.0 / math.sqrt(self.head_dim),
                  C.c_void_p(self.workspace_buffer.data_ptr()), self.workspace_buffer.numel(), self._stream_handle())
        tensors = (C.c_void_p(qc.data_ptr()), C.c_void_p(self.kv_caches[block_idx].data_ptr()), C.c_void_p(out.data_ptr()),
                   C.c_void_p(self_k.data_ptr()) if has_tail else None, C.c_void_p(self_v.data_ptr()) if has_tail else None,
                   C.c_void_p(self._kv_rows[ts].data_ptr()))
        if append_rows is not None:
            N.check(N.lib.lbm_attn_run_append(*tensors, C.c_void_p(append_rows.data_ptr()), self_k.shape[0], *common))
        elif self.device_token_counts:
            # the kernels read each stream's visible-token count from its table header, where the
            # last plan left it; the host's count above only sizes the launch
            live = self._tables[ts].data_ptr() + 4 * N.HDR["plan_kv_tokens"]
            N.check(N.lib.lbm_attn_run_live(*tensors, C.c_void_p(live), *common))
        else:
            N.check(N.lib.lbm_attn_run(*tensors, *common))
        return out

    def reset(self) -> None:
        """Reset all per-block state for a new sequence (flashinfer_cache.py:423-432).  What the
        device tables recorded about the sequence that ends here is raised first."""
        words = self._tables[:, :, N.HDR["error"]].cpu().tolist() if getattr(self, "_tables_live", False) else []
        ops = self._ops([{"ops": N.OP_RESET} for _ in range(self.num_streams)])
        for ts in range(self._n_sets):
            self._tables_step(ts, ops)
            self._counts[ts] = [_StreamCounts(self.max_patch_pages, self.max_special_pages)
                                for _ in range(self.num_streams)]
            self._plan_valid[ts] = False
            self._newest_self[ts] = False
            self._plan_tokens[ts] = [0] * self.num_streams
        for i in range(self.num_blocks):
            self.frame_count[i] = 0
            self._n_appends[i] = 0
        self._rows_log.clear()
        self._active = [True] * self.num_streams
        self._tables_live = True
        for ts, row in enumerate(words):      # the cache is reset either way
            for b, w in enumerate(row):
                self._raise_device_errors(w, ts, b)

    # ----- table read-back (synchronises; for tests, debugging and parity checks) -----
    def _read_tables(self, block_idx: int, stream: int):
        """Page ids and valid lengths of what `stream` sees, without the current frame's own
        rows.  Side-effect free: the plan runs into the page-table outputs only (the row table
        the blocks of the current frame attend through is not rewritten) and the two header
        words a plan publishes - the token count the kernels of a ``device_token_counts`` manager
        read, and the page count - are put back."""
        ts = self._set(block_idx)
        plan_words = slice(N.HDR["plan_kv_tokens"], N.HDR["plan_n_pages"] + 1)
        saved = self._tables[ts, :, plan_words].clone()
        per = [{"ops": N.OP_PLAN, "self_tokens": 0,
                "expect_kv_tokens": self._expect(self._visible_tokens(self._counts[ts][b]))}
               for b in range(self.num_streams)]
        self._tables_step(ts, self._ops(per), pages=True)
        hdr = self._tables[ts, stream, :N.HDR_WORDS].cpu().tolist()
        n_pages = hdr[N.HDR["plan_n_pages"]]
        lo = stream * self._pages_cap
        ids = self._page_ids[lo:lo + n_pages].cpu().tolist()
        lens = self._page_lens[lo:lo + n_pages].cpu().tolist()
        self._tables[ts, :, plan_words] = saved
        self._raise_device_errors(hdr[N.HDR["error"]], ts, stream)
        return hdr, ids, lens

    # ----- device-side error word -----
    @staticmethod
    def _raise_device_errors(word: int, ts: int, stream: int) -> None:
        if word:
            what = ", ".join(name for bit, name in N.TERR_NAMES.items() if word & bit)
            raise AssertionError(f"device page tables (set {ts}, stream {stream}) report: {what} "
                                 f"(error word 0x{word:x})")

    def check_device_errors(self) -> None:
        """Read the sticky error word of every stream's device tables (one small copy that
        waits for the queued work) and raise the reference's exception type for what it says:
        pool exhausted, rollback underflow (flashinfer_cache.py:276-278,290-293,489-494,
        533-537) or a visible-token count that disagrees with the host's.  The host's count
        mirror normally raises first; this is the check for paths where the mirror is advanced
        by book-keeping only (graph replay) or was bypassed.  Called by ``reset()``."""
        words = self._tables[:, :, N.HDR["error"]].cpu().tolist()
        for ts, row in enumerate(words):
            for b, w in enumerate(row):
                self._raise_device_errors(w, ts, b)

    def build_visible_page_table(self, block_idx: int, stream: int = 0) -> List[int]:
        """Page ids in order anchor, window, special/memory (flashinfer_cache.py:438-450)."""
        return self._read_tables(block_idx, stream)[1]

    def build_visible_page_lens(self, block_idx: int, stream: int = 0) -> List[int]:
        return self._read_tables(block_idx, stream)[2]

    def compute_last_page_len(self, block_idx: int, stream: int = 0) -> int:
        """Valid tokens in the last visible page (flashinfer_cache.py:452-470)."""
        _, ids, lens = self._read_tables(block_idx, stream)
        c = self._counts[self._set(block_idx)][stream]
        if self.layout == "two_stream" and c.n_special_pages == 0:
            return self._tpf - (self.pages_per_frame - 1) * self.page_size
        return lens[-1]

    def device_header(self, block_idx: int = 0, stream: int = 0) -> dict:
        hdr = self._tables[self._set(block_idx), stream, :N.HDR_WORDS].cpu().tolist()
        return {k: hdr[i] for k, i in N.HDR.items()}

    def append_rows(self, block_idx: int = 0) -> Tensor:
        """K row of every token of the latest append (-1 = not written)."""
        return self._append_rows[self._set(block_idx)]

    @property
    def num_frames(self) -> int:
        return self.frame_count[0] if self.frame_count else 0
