"""Dense (cache-less) attention of whole frames on the paged kernel.

The frame blocks of the aggregator attend within one frame (lingbot_map/layers/block.py:27-101,
lingbot_map/layers/attention.py:446-465: ``F.scaled_dot_product_attention`` over the frame's own
tokens).  The paged kernel covers that case with a trivial row table: every entry names a row
of the caller's own K/V, the pool is never read.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Dict, Tuple

import torch
from torch import Tensor

from . import _native as N

_plans: Dict[tuple, tuple] = {}          # (rows, streams, H, D, device) -> (row table, stream descriptors, workspace bytes)
_workspace: Dict[object, Tensor] = {}


def dense_attention(q: Tensor, k: Tensor, v: Tensor, num_streams: int = 1, q_prescaled: bool = False) -> Tensor:
    """softmax(q k^T / sqrt(D)) v for ``num_streams`` independent token groups.

    ``q``, ``k``, ``v``: ``[num_streams * n, H, D]`` contiguous, bf16 or fp32, on the GPU; group
    ``s`` is rows ``s * n .. (s + 1) * n - 1`` and attends to itself only.  Returns the same
    shape and dtype.  ``q_prescaled``: q already carries 1 / sqrt(D) and log2(e) (a producer run
    with ``q_scale = q_scale_log2(1 / sqrt(D))``).  Raises on anything the HIP kernels do not cover (there is no fallback)."""
    assert q.is_cuda and q.dim() == 3 and q.shape == k.shape == v.shape, "q, k, v: [tokens, H, D] on the GPU"
    assert q.dtype == k.dtype == v.dtype and q.dtype in (torch.bfloat16, torch.float32), "bf16 or fp32"
    rows, H, D = q.shape
    assert 1 <= num_streams <= N.MAX_STREAMS and rows % num_streams == 0
    n = rows // num_streams
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    key = (rows, num_streams, H, D, q.device)
    plan = _plans.get(key)
    if plan is None:
        # entry -1 - r names row r of the caller's own K/V
        kv_rows = (-1 - torch.arange(rows, dtype=torch.int32)).to(q.device)
        streams = (N.AttnStream * num_streams)(*[N.AttnStream(s * n, n, s * n, n) for s in range(num_streams)])
        need = int(N.lib.lbm_attn_workspace_bytes(streams, num_streams, H, D))
        plan = _plans[key] = (kv_rows, streams, need)
    kv_rows, streams, need = plan
    lane = (q.device, N.current_scratch_lane())     # one workspace per chain of launches that may overlap another
    ws = _workspace.get(lane)
    if ws is None or ws.numel() < max(need, 16):
        ws = torch.empty(max(int(need * 1.25), 1 << 20), dtype=torch.uint8, device=q.device)
        _workspace[lane] = ws
    out = torch.empty_like(q)
    p = lambda t: C.c_void_p(t.data_ptr())
    N.check(N.lib.lbm_attn_run(
        p(q), p(k), p(out), p(k), p(v), p(kv_rows), streams, num_streams, H, D, 16,
        N.DTYPE_BF16 if q.dtype == torch.bfloat16 else N.DTYPE_F32, 0.0 if q_prescaled else 1.0 / math.sqrt(D),
        p(ws), ws.numel(), N.stream_ptr(q.device)))
    return out
