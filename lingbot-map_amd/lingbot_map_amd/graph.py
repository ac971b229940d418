"""Replay of one streamed frame as a HIP graph.

The reference removes the per-frame launch overhead of its streaming loop by compiling the
blocks' pre- and post-attention pieces into CUDA graphs (gct_profile.py:40-57,
demo.py:181-186); its cache calls stay eager because their plans live on the host.  Here the
page tables live on the device and every launch of a steady-state frame has the same
arguments, so the whole frame - producer, table step, append, paged attention, the blocks'
PyTorch operations - is captured once and replayed.
"""
from __future__ import annotations

from typing import Callable, Sequence

import torch
from torch import Tensor


class GraphedFrame:
    """``frame_fn(*inputs) -> Tensor`` runs one streamed frame of every stream through all blocks
    (it calls the manager's ``step`` / ``step_qkv`` for each block).  The manager must be in
    ``steady_state`` (anchor and window full; evicted frames leaving no memory tokens unless the
    manager was built with ``device_token_counts=True``) and every frame replayed must be a
    keyframe; anything else has to go through the eager path.

    Calls overlap with nothing else on the manager: like the manager itself this is not
    re-entrant."""

    def __init__(self, manager, frame_fn: Callable[..., Tensor], example_inputs: Sequence[Tensor],
                 cross_frame_special: bool = True, camera_only: bool = False) -> None:
        if not manager.steady_state(cross_frame_special, camera_only):
            raise RuntimeError("GraphedFrame: the cache is not in a replayable steady state "
                               "(anchor and window full, no trajectory-memory growth, keyframes only)")
        self.manager = manager
        self._evict_args = (cross_frame_special, camera_only)
        self._inputs = [t.clone() for t in example_inputs]
        # one eager frame on a side stream first (library handles, workspaces, autotuning)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), torch.no_grad():
            frame_fn(*self._inputs)
        torch.cuda.current_stream().wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph), torch.no_grad():
            self._output = frame_fn(*self._inputs)
        # the capture ran the host side of one frame without executing it on the device
        manager.note_replayed_frames(-1, cross_frame_special, camera_only)
        if not manager.steady_state(cross_frame_special, camera_only):
            raise RuntimeError("GraphedFrame: the captured frame left the steady state")

    def __call__(self, *inputs: Tensor) -> Tensor:
        assert len(inputs) == len(self._inputs)
        for dst, src in zip(self._inputs, inputs):
            dst.copy_(src)
        self.graph.replay()
        self.manager.note_replayed_frames(1, *self._evict_args)
        return self._output
