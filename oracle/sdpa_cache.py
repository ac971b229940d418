"""CPU oracle: the arithmetic and the dict-cache semantics of the reference's SDPA path.

TEST INFRASTRUCTURE ONLY (see oracle/page_policy.py for who may import this package).

Restated from the reference (paths relative to its checkout):

* dense attention call, no mask, default scale 1/sqrt(D)
                                           lingbot_map/layers/attention.py:665-669
* paged -> dense bridge ("force_fp32" gather + SDPA)
                                           lingbot_map/layers/flashinfer_cache.py:324-347,372-383
* dict cache: append by concatenation on the frame axis
                                           lingbot_map/layers/attention.py:632-646
* dict cache eviction: keep the first ``scale`` and the last ``window`` frames, move the
  leading special tokens of the evicted frames to a side list, oldest first
                                           lingbot_map/layers/attention.py:676-718
* attended set = side list, then cached frames
                                           lingbot_map/layers/attention.py:652-663
* non-keyframe: attend to cache plus the current frame, store nothing
                                           lingbot_map/layers/attention.py:224-256
  (``SDPAAttention`` itself never reads the skip flag; the keyframe-gated set is the one
  the paged manager and ``CausalAttention`` define)

Parity pins (tests/test_oracle_attention.py): a float64 three-loop softmax on tiny shapes,
one KV token (output equals V), identical K rows (output equals the mean of V),
permutation invariance over KV tokens, and split-and-merge by log-sum-exp.
"""

from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------- arithmetic
def sdpa_nhd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, compute_dtype=torch.float32) -> torch.Tensor:
    """softmax(q k^T / sqrt(D)) v with tensors in ``[tokens, heads, head_dim]`` layout.

    Follows flashinfer_cache.py:379-383: permute to ``[1, H, tokens, D]``, call
    ``F.scaled_dot_product_attention`` with no mask and the default scale, permute back,
    cast to the dtype of ``q``."""
    q_b = q.to(compute_dtype).permute(1, 0, 2).unsqueeze(0)
    k_b = k.to(compute_dtype).permute(1, 0, 2).unsqueeze(0)
    v_b = v.to(compute_dtype).permute(1, 0, 2).unsqueeze(0)
    out = F.scaled_dot_product_attention(q_b, k_b, v_b)
    return out.squeeze(0).permute(1, 0, 2).to(q.dtype)


def naive_attention_f64(q: np.ndarray, k: np.ndarray, v: np.ndarray) -> np.ndarray:
    """Three explicit loops in float64; only for tiny shapes (pins ``sdpa_nhd``)."""
    tq, h, d = q.shape
    tk = k.shape[0]
    out = np.zeros((tq, h, d), dtype=np.float64)
    scale = 1.0 / math.sqrt(d)
    for i in range(tq):
        for hh in range(h):
            scores = [scale * float(np.dot(q[i, hh].astype(np.float64), k[j, hh].astype(np.float64))) for j in range(tk)]
            mx = max(scores)
            w = [math.exp(s - mx) for s in scores]
            z = sum(w)
            for j in range(tk):
                out[i, hh] += (w[j] / z) * v[j, hh].astype(np.float64)
    return out


def gather_paged(
    pool: torch.Tensor, page_ids: Sequence[int], page_lens: Sequence[int]
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dense ``[kv_len, H, D]`` K and V from a ``[pages, 2, page_size, H, D]`` pool
    (flashinfer_cache.py:339-346, with a valid length per page instead of only the last)."""
    ks = [pool[p, 0, :n] for p, n in zip(page_ids, page_lens)]
    vs = [pool[p, 1, :n] for p, n in zip(page_ids, page_lens)]
    return torch.cat(ks, dim=0), torch.cat(vs, dim=0)


def write_frame(pool: torch.Tensor, plan_pages: Sequence[int], plan_slots: Sequence[int], k: torch.Tensor, v: torch.Tensor) -> None:
    """Store one frame token by token (flashinfer_cache.py:504-505,548-549; cast to the
    pool dtype as in :215-218)."""
    pages = torch.as_tensor(list(plan_pages), dtype=torch.long)
    slots = torch.as_tensor(list(plan_slots), dtype=torch.long)
    pool[pages, 0, slots] = k.to(pool.dtype)
    pool[pages, 1, slots] = v.to(pool.dtype)


# --------------------------------------------------------------------------- dict cache
class DictCacheOracle:
    """Frame-list restatement of the SDPA backend's per-block KV cache.

    ``frames`` plays the role of ``kv_cache["k_i"]``/``["v_i"]`` (frame axis = list index),
    ``special`` that of ``kv_cache["k_i_special"]``/``["v_i_special"]``."""

    def __init__(
        self,
        scale_frames: int,
        sliding_window: int,
        num_special_tokens: int,
        cross_frame_special: bool = True,
        include_scale_frames: bool = True,
        camera_only: bool = False,
    ):
        self.scale_frames = scale_frames
        self.sliding_window = sliding_window
        self.num_special_tokens = num_special_tokens
        self.cross_frame_special = cross_frame_special
        self.include_scale_frames = include_scale_frames
        self.camera_only = camera_only
        self.frames: List[Tuple[torch.Tensor, torch.Tensor]] = []
        self.special: List[Tuple[torch.Tensor, torch.Tensor]] = []

    def reset(self) -> None:
        self.frames, self.special = [], []

    def _evict(self) -> None:
        n = len(self.frames)
        if n <= self.sliding_window + self.scale_frames:
            return
        start, end = self.scale_frames, n - self.sliding_window
        if end <= start:
            return
        if self.cross_frame_special:
            keep = 1 if self.camera_only else self.num_special_tokens
            for k, v in self.frames[start:end]:
                self.special.append((k[:keep].clone(), v[:keep].clone()))
        tail = self.frames[n - self.sliding_window:]
        self.frames = (self.frames[: self.scale_frames] + tail) if self.include_scale_frames else tail

    def visible(self, k: torch.Tensor, v: torch.Tensor, keyframe: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
        """Advance by one frame and return the dense K, V the frame attends to."""
        if keyframe:
            self.frames.append((k, v))
            self._evict()
            frames = self.frames
        else:
            frames = self.frames + [(k, v)]
        ks = [s[0] for s in self.special] + [f[0] for f in frames]
        vs = [s[1] for s in self.special] + [f[1] for f in frames]
        return torch.cat(ks, dim=0), torch.cat(vs, dim=0)

    def step(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, keyframe: bool = True, compute_dtype=torch.float32) -> torch.Tensor:
        kk, vv = self.visible(k, v, keyframe)
        return sdpa_nhd(q, kk, vv, compute_dtype)


# --------------------------------------------------------------------------- paged stream
class PagedStreamOracle:
    """One block of one stream: page policy + a CPU page pool + gather/SDPA attention.

    The call sequence mirrors the reference's global block
    (lingbot_map/layers/block.py:256-278): keyframe = append, evict, attend;
    non-keyframe = defer eviction, append, attend, roll back."""

    def __init__(self, policy, num_heads: int, head_dim: int, dtype=torch.float32):
        self.policy = policy
        self.pool = torch.zeros(
            policy.page_base + policy.max_num_pages, 2, policy.page_size, num_heads, head_dim, dtype=dtype
        )

    def append_frame(self, k: torch.Tensor, v: torch.Tensor):
        plan = self.policy.append_frame()
        write_frame(self.pool, plan.page, plan.slot, k, v)
        return plan

    def compute_attention(self, q: torch.Tensor, compute_dtype=torch.float32) -> torch.Tensor:
        if self.policy.frame_count == 0:  # flashinfer_cache.py:368-370
            return torch.zeros_like(q)
        kk, vv = gather_paged(self.pool, self.policy.build_visible_page_table(), self.policy.build_visible_page_lens())
        return sdpa_nhd(q.to(self.pool.dtype), kk, vv, compute_dtype)

    def step(self, q, k, v, keyframe: bool = True, compute_dtype=torch.float32, **evict_kw) -> torch.Tensor:
        pol = self.policy
        if keyframe:
            self.append_frame(k, v)
            pol.evict_frames(pol.scale_frames, pol.sliding_window, **evict_kw)
            return self.compute_attention(q, compute_dtype)
        prev = pol._defer_eviction
        pol._defer_eviction = True
        self.append_frame(k, v)
        out = self.compute_attention(q, compute_dtype)
        pol.rollback_last_frame()
        pol._defer_eviction = prev
        return out


def merge_splits(outs: Sequence[torch.Tensor], lses: Sequence[torch.Tensor]) -> torch.Tensor:
    """Combine attention over disjoint KV subsets from their normalised outputs and
    natural-log sum-exps (``[tokens, heads]``)."""
    lse = torch.stack(list(lses), dim=0)
    w = torch.softmax(lse, dim=0).unsqueeze(-1)
    return (w * torch.stack(list(outs), dim=0)).sum(dim=0)


def attention_with_lse(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    s = torch.einsum("qhd,khd->hqk", q.double(), k.double()) / math.sqrt(q.shape[-1])
    lse = torch.logsumexp(s, dim=-1)
    out = torch.einsum("hqk,khd->qhd", torch.softmax(s, dim=-1), v.double())
    return out, lse.transpose(0, 1)
