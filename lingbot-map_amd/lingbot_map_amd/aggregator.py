"""Streaming aggregator shell on the HIP cache path.

``HipAggregatorStream`` stands next to the reference's ``AggregatorStream``
(lingbot_map/aggregator/stream.py:37-529 on ``AggregatorBase``, lingbot_map/aggregator/base.py:56-606):
the same constructor vocabulary, the same parameter names for the special tokens
(``camera_token``, ``register_token``, ``scale_token``: ``[1, 2, n, C]`` with index 0 for the
first frame(s) and index 1 for the rest), ``frame_blocks`` / ``global_blocks`` module lists, and
the same ``forward(images) -> (list of [B, S, P, 2C], patch_start_idx)``:

* images are normalised, patch-embedded and prefixed with the special tokens (base.py:335-395);
* ``depth / aa_block_size`` groups alternate frame attention (every frame on its own,
  ``[B * S, P, C]``, 2-D rotary embedding; base.py:444-500) and global attention (the streamed
  frame against the paged KV cache, ``[B, S * P, C]``; stream.py:415-529);
* each group's frame and global outputs are concatenated on the channel axis (base.py:600-604).

What differs from the reference: the batch axis carries independent *streams* (each with its
own window; one manager serves them all as one ragged batch), the global blocks are
``HipPagedBlock``s driving a ``HipPagedKVCacheManager``, and the image encoder is a parameter
(``"conv"``: a patch convolution; ``"vit"``: the convolution followed by a trunk of plain
blocks and a LayerNorm, the shape of the DINOv2 encoder without its position table and
pre-processing; or any module that returns ``[B * S, patches, C]``).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple, Union

import torch
from torch import Tensor, nn

from .block import (HipPagedBlock, PositionGetter, RotaryPositionEmbedding2D, RotaryPositionEmbedding3D)
from .manager import HipPagedKVCacheManager

_RESNET_MEAN = (0.485, 0.456, 0.406)
_RESNET_STD = (0.229, 0.224, 0.225)


class PatchConv(nn.Module):
    """Image to patch tokens by one strided convolution (the reference's ``"conv"`` patch
    embedding, lingbot_map/aggregator/base.py:190-197)."""

    def __init__(self, patch_size: int, embed_dim: int) -> None:
        super().__init__()
        self.proj = nn.Conv2d(3, embed_dim, kernel_size=patch_size, stride=patch_size)

    def forward(self, images: Tensor) -> Tensor:          # [N, 3, H, W] -> [N, patches, C]
        return self.proj(images).flatten(2).transpose(1, 2)


class PatchTrunk(nn.Module):
    """Patch convolution, a trunk of plain transformer blocks and a final LayerNorm: the cost
    shape of the reference's DINOv2 ViT encoder (lingbot_map/layers/vision_transformer.py:383-394)
    without its learned position table, class / register tokens and weights."""

    def __init__(self, patch_size: int, embed_dim: int, depth: int, num_heads: int, mlp_ratio: float) -> None:
        super().__init__()
        self.conv = PatchConv(patch_size, embed_dim)
        self.blocks = nn.ModuleList([HipPagedBlock(dim=embed_dim, num_heads=num_heads, mlp_ratio=mlp_ratio, init_values=1.0)
                                     for _ in range(depth)])
        self.norm = nn.LayerNorm(embed_dim)

    def forward(self, images: Tensor) -> Tensor:
        x = self.conv(images)
        normed = None
        for i, blk in enumerate(self.blocks):   # each block hands the next one its norm1 (or the final norm)
            nxt = self.blocks[i + 1].norm1 if i + 1 < len(self.blocks) else self.norm
            x, normed = blk(x, normed=normed, next_norm=nxt)
        return normed if torch.is_tensor(normed) else self.norm(x)   # (row statistics: nobody left to fold them)


def _first_then_rest(token: Tensor, first: Tensor) -> Tensor:
    """``token`` ``[1, 2, n, C]``, ``first`` bool ``[frames]`` -> ``[frames, n, C]``: index 0 of the
    pair where ``first`` holds, index 1 elsewhere (slice_expand_and_flatten, base.py:24-53)."""
    return torch.where(first.view(-1, 1, 1), token[0, 0].unsqueeze(0), token[0, 1].unsqueeze(0))


class HipAggregatorStream(nn.Module):
    def __init__(
        self,
        img_size: int = 518,
        patch_size: int = 14,
        embed_dim: int = 1024,
        depth: int = 24,
        num_heads: int = 16,
        mlp_ratio: float = 4.0,
        num_register_tokens: int = 4,
        qkv_bias: bool = True,
        proj_bias: bool = True,
        ffn_bias: bool = True,
        qk_norm: bool = True,
        init_values: float = 0.01,
        patch_embed: Union[str, nn.Module] = "conv",
        aa_order: Sequence[str] = ("frame", "global"),
        aa_block_size: int = 1,
        rope_freq: float = 100,
        disable_global_rope: bool = False,
        num_frame_for_scale: int = 1,
        enable_3d_rope: bool = False,
        max_frame_num: int = 1024,
        kv_cache_sliding_window: Union[int, Sequence[int]] = 64,
        kv_cache_scale_frames: int = 8,
        kv_cache_cross_frame_special: bool = True,
        kv_cache_include_scale_frames: bool = True,
        kv_cache_camera_only: bool = False,
        kv_cache_force_fp32: bool = False,
        *,
        use_scale_token: bool = True,
        page_size: Optional[int] = None,
        layout: str = "two_stream",
        num_streams: int = 1,
        encoder_depth: int = 24,
        device_token_counts: bool = False,
    ) -> None:
        super().__init__()
        if depth % aa_block_size != 0:
            raise ValueError(f"depth ({depth}) must be divisible by aa_block_size ({aa_block_size})")
        for kind in aa_order:
            if kind not in ("frame", "global"):
                raise ValueError(f"Unknown attention type: {kind}")
        windows = list(kv_cache_sliding_window) if isinstance(kv_cache_sliding_window, (list, tuple)) else None
        if windows is not None and len(windows) != num_streams:
            raise ValueError("one kv_cache_sliding_window per stream")
        self.img_size, self.patch_size, self.embed_dim, self.depth = img_size, patch_size, embed_dim, depth
        self.num_heads, self.mlp_ratio, self.num_register_tokens = num_heads, mlp_ratio, num_register_tokens
        self.aa_order, self.aa_block_size, self.aa_block_num = tuple(aa_order), aa_block_size, depth // aa_block_size
        self.disable_global_rope = disable_global_rope
        self.num_frame_for_scale = num_frame_for_scale
        self.enable_3d_rope, self.max_frame_num = enable_3d_rope, max_frame_num
        self.kv_cache_sliding_window = kv_cache_sliding_window
        self.kv_cache_scale_frames = kv_cache_scale_frames
        self.kv_cache_cross_frame_special = kv_cache_cross_frame_special
        self.kv_cache_include_scale_frames = kv_cache_include_scale_frames
        self.kv_cache_camera_only = kv_cache_camera_only
        self.kv_cache_force_fp32 = kv_cache_force_fp32
        self.use_scale_token = use_scale_token
        self.page_size, self.layout, self.num_streams = page_size, layout, num_streams
        self.device_token_counts = device_token_counts

        if isinstance(patch_embed, nn.Module):
            self.patch_embed = patch_embed
        elif patch_embed == "conv":
            self.patch_embed = PatchConv(patch_size, embed_dim)
        elif patch_embed == "vit":
            self.patch_embed = PatchTrunk(patch_size, embed_dim, encoder_depth, num_heads, mlp_ratio)
        else:
            raise NotImplementedError(f"Unknown patch_embed type: {patch_embed}")

        self.rope = RotaryPositionEmbedding2D(frequency=rope_freq) if rope_freq > 0 else None
        self.position_getter = PositionGetter() if self.rope is not None else None
        block = dict(dim=embed_dim, num_heads=num_heads, mlp_ratio=mlp_ratio, qkv_bias=qkv_bias, proj_bias=proj_bias,
                     ffn_bias=ffn_bias, init_values=init_values, qk_norm=qk_norm)
        window = max(windows) if windows is not None else kv_cache_sliding_window
        self.frame_blocks = nn.ModuleList([HipPagedBlock(**block, rope=self.rope) for _ in range(depth)])
        self.global_blocks = nn.ModuleList([
            HipPagedBlock(**block, rope=self.rope if not disable_global_rope else None,
                          kv_cache_sliding_window=window, kv_cache_scale_frames=kv_cache_scale_frames,
                          kv_cache_cross_frame_special=kv_cache_cross_frame_special,
                          kv_cache_include_scale_frames=kv_cache_include_scale_frames,
                          kv_cache_camera_only=kv_cache_camera_only)
            for _ in range(depth)])

        # special tokens (stream.py:151-177): camera, registers and - in the reference always - scale
        self.camera_token = nn.Parameter(torch.randn(1, 2, 1, embed_dim))
        nn.init.normal_(self.camera_token, std=1e-6)
        if num_register_tokens > 0:
            self.register_token = nn.Parameter(torch.randn(1, 2, num_register_tokens, embed_dim))
            nn.init.normal_(self.register_token, std=1e-6)
        if use_scale_token:
            self.scale_token = nn.Parameter(torch.ones(1, 2, 1, embed_dim))
            nn.init.normal_(self.scale_token, std=1e-6)
        self.num_special_tokens = 1 + num_register_tokens + (1 if use_scale_token else 0)
        self.patch_start_idx = self.num_special_tokens
        self.register_buffer("_resnet_mean", torch.tensor(_RESNET_MEAN).view(1, 1, 3, 1, 1), persistent=False)
        self.register_buffer("_resnet_std", torch.tensor(_RESNET_STD).view(1, 1, 3, 1, 1), persistent=False)

        self.rope3d = None
        if enable_3d_rope:   # stream.py:256-271
            self.rope3d = RotaryPositionEmbedding3D(attention_head_dim=embed_dim // num_heads,
                                                    patch_size=(1, patch_size, patch_size), max_seq_len=max_frame_num)
        self.kv_cache_manager: Optional[HipPagedKVCacheManager] = None     # built on the first forward
        self.total_frames_processed = 0
        self._cached_pos3d = None

    # ------------------------------------------------------------------ cache
    def _get_manager(self, device, dtype, tokens_per_frame: int) -> HipPagedKVCacheManager:
        """The cache manager, sized on first use (stream.py:198-234)."""
        if self.kv_cache_manager is None:
            windows = self.kv_cache_sliding_window
            widest = max(windows) if isinstance(windows, (list, tuple)) else windows
            self.kv_cache_manager = HipPagedKVCacheManager(
                num_blocks=self.depth, max_num_frames=self.kv_cache_scale_frames + widest + 16,
                tokens_per_frame=tokens_per_frame, num_heads=self.num_heads, head_dim=self.embed_dim // self.num_heads,
                dtype=dtype, device=device, num_special_tokens=self.num_special_tokens,
                scale_frames=self.kv_cache_scale_frames,
                sliding_window=list(windows) if isinstance(windows, (list, tuple)) else windows,
                max_total_frames=self.max_frame_num + 100, force_fp32=self.kv_cache_force_fp32,
                page_size=self.page_size, layout=self.layout, num_streams=self.num_streams,
                device_token_counts=self.device_token_counts)
        return self.kv_cache_manager

    def clean_kv_cache(self) -> None:
        """Start a new sequence (stream.py:236-249)."""
        if self.kv_cache_manager is not None:
            self.kv_cache_manager.reset()
        self.total_frames_processed = 0
        self._cached_pos3d = None

    # ------------------------------------------------------------------ embedding
    def _prepare_special_tokens(self, B: int, S: int, C: int, num_frame_for_scale: Optional[int] = None) -> Tensor:
        """``[B * S, num_special, C]``: the first frame of a sequence takes index 0 of the camera
        and register pairs, the first ``num_frame_for_scale`` frames index 0 of the scale pair;
        frames are counted from the number already cached (stream.py:297-368)."""
        scale_frames = self.num_frame_for_scale if num_frame_for_scale is None else num_frame_for_scale
        cached = self.kv_cache_manager.num_frames if self.kv_cache_manager is not None else 0
        # which frames of the call are "first" is host knowledge; the assembled tokens of a pattern
        # are kept until a parameter changes (every steady-state frame asks for the same ones)
        first = tuple(cached + i < 1 for i in range(S))
        first_scale = tuple(cached + i < max(min(scale_frames, cached + S), 1) for i in range(S))
        params = [self.camera_token] + ([self.register_token] if self.num_register_tokens > 0 else []) + \
                 ([self.scale_token] if self.use_scale_token else [])
        key = (B, first, first_scale, tuple((t._version, t.data_ptr(), t.dtype) for t in params))
        hit = self.__dict__.get("_special_cache")
        if hit is not None and hit[0] == key and not torch.is_grad_enabled():
            return hit[1]
        index = cached + torch.arange(S, device=self.camera_token.device)
        parts = [_first_then_rest(self.camera_token, index < 1)]
        if self.num_register_tokens > 0:
            parts.append(_first_then_rest(self.register_token, index < 1))
        if self.use_scale_token:
            parts.append(_first_then_rest(self.scale_token, index < max(min(scale_frames, cached + S), 1)))
        tokens = torch.cat(parts, dim=1)                                   # [S, n, C]
        tokens = tokens.unsqueeze(0).expand(B, -1, -1, -1).reshape(B * S, self.num_special_tokens, C)
        if not torch.is_grad_enabled():
            self.__dict__["_special_cache"] = (key, tokens)
        return tokens

    def _embed_images(self, images: Tensor, num_frame_for_scale: Optional[int] = None):
        B, S, c_in, H, W = images.shape
        if c_in != 3:
            raise ValueError(f"Expected 3 input channels, got {c_in}")
        if B != self.num_streams:
            raise ValueError(f"images carry {B} streams, the aggregator was built for {self.num_streams}")
        images = (images - self._resnet_mean.to(images.dtype)) / self._resnet_std.to(images.dtype)
        patches = self.patch_embed(images.view(B * S, c_in, H, W))
        if isinstance(patches, dict):
            patches = patches["x_norm_patchtokens"]
        C = patches.shape[-1]
        special = self._prepare_special_tokens(B, S, C, num_frame_for_scale).to(patches.dtype)
        tokens = torch.cat([special, patches], dim=1)
        return tokens, B, S, tokens.shape[1], C

    def _get_positions(self, frames: int, H: int, W: int, device) -> Optional[Tensor]:
        """(y, x) of every token, ``[frames, P, 2]``: specials at (0, 0), patches on the grid
        shifted by one (base.py:416-440)."""
        if self.rope is None:
            return None
        key = (frames, H, W, str(device))
        hit = self.__dict__.get("_positions_cache")
        if hit is not None and hit[0] == key:      # the same tensor again: the rotary table derived from it is reused too
            return hit[1]
        pos = self.position_getter(frames, H // self.patch_size, W // self.patch_size, device=device) + 1
        zeros = torch.zeros(frames, self.patch_start_idx, 2, dtype=pos.dtype, device=device)
        pos = torch.cat([zeros, pos], dim=1)
        self.__dict__["_positions_cache"] = (key, pos)
        return pos

    # ------------------------------------------------------------------ forward
    def stream_table(self, frames: int, H: int, W: int, device, first_frame: Optional[int] = None) -> Optional[Tensor]:
        """Rotary table of the global blocks for ``frames`` frames starting at stream index
        ``first_frame`` (default: the frames streamed so far), complex ``[1, 1, frames * P, D / 2]``
        (stream.py:273-295); None without the 3-D embedding."""
        if self.rope3d is None:
            return None
        f0 = self.total_frames_processed if first_frame is None else first_frame
        return self.rope3d(ppf=frames, pph=H // self.patch_size, ppw=W // self.patch_size,
                           patch_start_idx=self.num_special_tokens, device=device, f_start=f0, f_end=f0 + frames)

    def forward(self, images: Tensor, selected_idx: Optional[List[int]] = None,
                num_frame_for_scale: Optional[int] = None, sliding_window_size: Optional[int] = None,
                num_frame_per_block: int = 1, *, pos3d: Optional[Tensor] = None,
                tokens: Optional[Tensor] = None) -> Tuple[List[Tensor], int]:
        """``images`` ``[streams, S, 3, H, W]`` in [0, 1]; ``S`` is 1 in streaming (more only for
        the anchor pass of a single stream).  Returns the groups' outputs ``[streams, S, P, 2C]``
        (all groups, or those in ``selected_idx``) and the index of the first patch token.
        ``pos3d``: the global blocks' rotary table of this call, for a caller that keeps the frame
        index itself (graph replay); the stream's frame counter is then left alone.
        ``tokens``: what ``_embed_images`` returned for these images, ``[streams * S, P, C]``, for
        a caller that ran the image encoder ahead of time; ``images`` then only gives the sizes."""
        H, W = images.shape[-2:]
        if tokens is None:
            tokens, B, S, P, C = self._embed_images(images, num_frame_for_scale)
        else:
            (B, S), (P, C) = images.shape[:2], tokens.shape[-2:]
        pos = self._get_positions(B * S, H, W, images.device)
        manager = self._get_manager(tokens.device, tokens.dtype, P)
        scale_frames = self.num_frame_for_scale if num_frame_for_scale is None else num_frame_for_scale
        frame_idx = global_idx = 0
        outputs: List[Tensor] = []
        # the blocks in the order they run: each one's last residual kernel also applies the norm1
        # of the block after it, so only the first block of a call launches a LayerNorm of its own
        order = [blocks[i] for g in range(self.aa_block_num) for kind, blocks in
                 ((k, self.frame_blocks if k == "frame" else self.global_blocks) for k in self.aa_order)
                 for i in range(g * self.aa_block_size, (g + 1) * self.aa_block_size)]
        step, normed = 0, None

        def run(block, tokens, normed, **kw):
            nonlocal step
            nxt = order[step + 1].norm1 if step + 1 < len(order) else None
            assert order[step] is block
            step += 1
            if nxt is None:
                return block(tokens, normed=normed, **kw), None
            return block(tokens, normed=normed, next_norm=nxt, **kw)

        for group in range(self.aa_block_num):
            frame_out: List[Tensor] = []
            global_out: List[Tensor] = []
            for kind in self.aa_order:
                if kind == "frame":
                    tokens = tokens.reshape(B * S, P, C)
                    normed = normed.reshape(B * S, P, C) if torch.is_tensor(normed) else normed
                    for _ in range(self.aa_block_size):
                        tokens, normed = run(self.frame_blocks[frame_idx], tokens, normed, pos=pos)
                        frame_idx += 1
                        frame_out.append(tokens.view(B, S, P, C))
                else:
                    tokens = tokens.reshape(B, S * P, C)
                    normed = normed.reshape(B, S * P, C) if torch.is_tensor(normed) else normed
                    first_group = global_idx < self.aa_block_size
                    if self.rope3d is not None:     # frame index = frames streamed so far (stream.py:464-478)
                        if first_group:
                            self._cached_pos3d = pos3d if pos3d is not None else self.stream_table(S, H, W, tokens.device)
                        pos_g = self._cached_pos3d
                    else:
                        pos_g = pos.view(B, S * P, 2) if pos is not None else None
                    for _ in range(self.aa_block_size):
                        tokens, normed = run(
                            self.global_blocks[global_idx], tokens, normed,
                            pos=pos_g, num_patches=P - self.num_special_tokens, num_special=self.num_special_tokens,
                            num_frames=S, enable_3d_rope=self.rope3d is not None, kv_cache=manager, global_idx=global_idx,
                            num_frame_per_block=num_frame_per_block, num_frame_for_scale=scale_frames,
                            num_register_tokens=self.num_register_tokens)
                        global_idx += 1
                        global_out.append(tokens.view(B, S, P, C))
                    if first_group and pos3d is None and not getattr(manager, "_skip_append", False):
                        self.total_frames_processed += S
            if selected_idx is None or group in selected_idx:
                for f, g in zip(frame_out, global_out):
                    outputs.append(torch.cat([f, g], dim=-1))
        return outputs, self.patch_start_idx


class GraphedAggregator:
    """One streamed frame of every stream through the whole aggregator as HIP graphs, one for
    keyframes and one for read-only frames (the reference's counterpart is its compile recipe,
    gct_profile.py:40-57, which covers every frame of the stream).  The cache must be in its
    steady state (``HipPagedKVCacheManager.steady_state``).  The rotary table of the global
    blocks depends on the frame index, so it is a graph input: it is computed eagerly for each
    call and copied into the captured buffer.

    ``graphed(images, keyframe=True) -> [groups, streams, 1, P, 2C]`` for ``images``
    ``[streams, 1, 3, H, W]``; the result buffer is overwritten by the next call of the same kind."""

    def __init__(self, model: HipAggregatorStream, example_images: Tensor,
                 selected_idx: Optional[List[int]] = None) -> None:
        from .graph import GraphedStream
        if model.kv_cache_manager is None:
            raise RuntimeError("GraphedAggregator: stream the anchor and window frames eagerly first")
        self.model = model
        self._hw = tuple(example_images.shape[-2:])
        dev = example_images.device

        def frame_fn(images: Tensor, table: Optional[Tensor] = None) -> Tensor:
            pos3d = torch.view_as_complex(table) if table is not None else None
            outs, _ = model(images, selected_idx=selected_idx, pos3d=pos3d)
            return torch.stack(outs)

        inputs = [example_images]
        if model.rope3d is not None:
            inputs.append(self._table(dev))
        self.stream = GraphedStream(model.kv_cache_manager, frame_fn, inputs, model.kv_cache_cross_frame_special,
                                    model.kv_cache_camera_only)

    def _table(self, device) -> Tensor:
        t = self.model.stream_table(1, self._hw[0], self._hw[1], device)
        return torch.view_as_real(t.to(torch.complex64)).contiguous()

    def __call__(self, images: Tensor, keyframe: bool = True) -> Tensor:
        assert tuple(images.shape[-2:]) == self._hw, "the graphs were captured for another image size"
        extra = [self._table(images.device)] if self.model.rope3d is not None else []
        out = self.stream(images, *extra, keyframe=keyframe)
        if keyframe:
            self.model.total_frames_processed += 1
        return out


class PipelinedAggregator:
    """Steady-state streaming with one frame of look-ahead.  The image encoder (normalisation,
    patch convolution, encoder blocks, special tokens: ``_embed_images``) reads nothing of the
    cache, so the encoder of frame t + 1 does not depend on the frame and global blocks of frame
    t.  Here the two are branches of one HIP graph on two streams: one frame's kernels leave CUs
    idle (128 to 192 workgroups of a GEMM on 256 CUs, the gaps between dependent launches) which
    the other branch's kernels fill.  Results are those of ``GraphedAggregator`` bit for bit; what
    changes is when an image must be there: a call hands in the NEXT frame's images and returns
    the outputs of the frame handed in by the call before (``prime`` hands in the first).

    The encoder branch runs under ``scratch_lane(1)``, i.e. on scratch memory of its own.  The cache
    must be in its steady state, as for ``GraphedAggregator``."""

    def __init__(self, model: HipAggregatorStream, example_images: Tensor,
                 selected_idx: Optional[List[int]] = None) -> None:
        from . import _native as N
        from .graph import GraphedStream
        if model.kv_cache_manager is None:
            raise RuntimeError("PipelinedAggregator: stream the anchor and window frames eagerly first")
        self.model = model
        self._hw = tuple(example_images.shape[-2:])
        self._side = torch.cuda.Stream()
        self._primed = False
        dev = example_images.device
        with torch.no_grad():
            self._next = torch.empty_like(model._embed_images(example_images)[0])   # tokens of the frame in waiting

        def frame_fn(images_next: Tensor, table: Optional[Tensor] = None) -> Tensor:
            main = torch.cuda.current_stream()
            current = self._next.clone()
            self._side.wait_stream(main)          # fork: the encoder may overwrite the buffer from here on
            with torch.cuda.stream(self._side), N.scratch_lane(1):
                self._next.copy_(model._embed_images(images_next)[0])
            pos3d = torch.view_as_complex(table) if table is not None else None
            outs, _ = model(images_next, selected_idx=selected_idx, pos3d=pos3d, tokens=current)
            out = torch.stack(outs)
            main.wait_stream(self._side)          # join
            return out

        inputs = [example_images]
        if model.rope3d is not None:
            inputs.append(self._table(dev))
        self.stream = GraphedStream(model.kv_cache_manager, frame_fn, inputs, model.kv_cache_cross_frame_special,
                                    model.kv_cache_camera_only)

    def _table(self, device) -> Tensor:
        t = self.model.stream_table(1, self._hw[0], self._hw[1], device)
        return torch.view_as_real(t.to(torch.complex64)).contiguous()

    @torch.no_grad()
    def prime(self, images: Tensor) -> None:
        """Encode the first frame of the pipeline (eagerly); its outputs come out of the next call."""
        assert tuple(images.shape[-2:]) == self._hw, "the graphs were captured for another image size"
        self._next.copy_(self.model._embed_images(images)[0])
        self._primed = True

    def __call__(self, next_images: Tensor, keyframe: bool = True) -> Tensor:
        """Outputs ``[groups, streams, 1, P, 2C]`` of the frame in waiting (a keyframe or not), while
        ``next_images`` are encoded and take its place.  The result buffer is overwritten by the next
        call of the same kind."""
        if not self._primed:
            raise RuntimeError("PipelinedAggregator: prime() the first frame before the first call")
        assert tuple(next_images.shape[-2:]) == self._hw, "the graphs were captured for another image size"
        extra = [self._table(next_images.device)] if self.model.rope3d is not None else []
        out = self.stream(next_images, *extra, keyframe=keyframe)
        if keyframe:
            self.model.total_frames_processed += 1
        return out
