"""Replay of one streamed frame as a HIP graph.

The reference removes the per-frame launch overhead of its streaming loop by compiling the
blocks' pre- and post-attention pieces into CUDA graphs (gct_profile.py:40-57,
demo.py:181-186); its cache calls stay eager because their plans live on the host.  Here the
page tables live on the device and every launch of a steady-state frame has the same
arguments, so the whole frame - producer, table step, append, paged attention, the blocks'
PyTorch operations - is captured once and replayed; a frame that only reads the cache (a
non-keyframe) changes no table at all and gets a graph of its own.
"""
from __future__ import annotations

from typing import Callable, Sequence

import torch
from torch import Tensor


class GraphedFrame:
    """``frame_fn(*inputs) -> Tensor`` runs one streamed frame of every stream through all blocks
    (it calls the manager's ``step`` / ``step_qkv`` for each block, with ``keyframe=None`` so that
    the manager's ``_skip_append`` switch decides).  The manager must be in ``steady_state``
    (anchor and window full; evicted frames leaving no memory tokens unless the manager was built
    with ``device_token_counts=True``).

    ``read_only=False`` captures a keyframe (append, evict, attend), ``read_only=True`` a frame
    that attends to the cache plus itself and stores nothing; a captured graph replays only
    frames of its own kind.  Construction runs ``frame_fn`` once eagerly on ``example_inputs``
    as a read-only frame (library handles, workspaces, autotuning) and once under capture;
    neither changes the cache, the tables or the host's counts, and the outputs of both are
    discarded - ``example_inputs`` only have to have the right shapes and dtypes.

    Calls overlap with nothing else on the manager: like the manager itself this is not
    re-entrant."""

    def __init__(self, manager, frame_fn: Callable[..., Tensor], example_inputs: Sequence[Tensor],
                 cross_frame_special: bool = True, camera_only: bool = False, read_only: bool = False) -> None:
        if not manager.steady_state(cross_frame_special, camera_only):
            raise RuntimeError("GraphedFrame: the cache is not in a replayable steady state "
                               "(anchor and window full, no trajectory-memory growth)")
        self.manager = manager
        self.read_only = bool(read_only)
        self._evict_args = (cross_frame_special, camera_only)
        self._inputs = [t.clone() for t in example_inputs]
        skip_before = manager._skip_append
        try:
            # one eager read-only frame on a side stream first: nothing is stored, nothing evicted
            manager._skip_append = True
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side), torch.no_grad():
                frame_fn(*self._inputs)
            torch.cuda.current_stream().wait_stream(side)
            manager._skip_append = self.read_only
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph), torch.no_grad():
                self._output = frame_fn(*self._inputs)
        finally:
            manager._skip_append = skip_before
        if not self.read_only:
            # the capture ran the host side of one keyframe without executing it on the device
            manager.note_replayed_frames(-1, cross_frame_special, camera_only)
        if not manager.steady_state(cross_frame_special, camera_only):
            raise RuntimeError("GraphedFrame: the captured frame left the steady state")

    def __call__(self, *inputs: Tensor) -> Tensor:
        assert len(inputs) == len(self._inputs)
        for dst, src in zip(self._inputs, inputs):
            dst.copy_(src)
        self.graph.replay()
        if not self.read_only:
            self.manager.note_replayed_frames(1, *self._evict_args)
        return self._output


class GraphedStream:
    """Both graphs of a steady-state stream: ``stream(*inputs, keyframe=True)`` replays the
    keyframe graph, ``keyframe=False`` the read-only one - the keyframe-interval driver
    (lingbot_map/models/gct_stream.py:446-464) without an eager frame in between.  The outputs
    of the two graphs live in different buffers; each is overwritten by the next replay of its
    own graph."""

    def __init__(self, manager, frame_fn: Callable[..., Tensor], example_inputs: Sequence[Tensor],
                 cross_frame_special: bool = True, camera_only: bool = False) -> None:
        self.keyframe = GraphedFrame(manager, frame_fn, example_inputs, cross_frame_special, camera_only)
        self.read_only = GraphedFrame(manager, frame_fn, example_inputs, cross_frame_special, camera_only,
                                      read_only=True)

    def __call__(self, *inputs: Tensor, keyframe: bool = True) -> Tensor:
        return (self.keyframe if keyframe else self.read_only)(*inputs)
