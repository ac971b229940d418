"""Global-attention block on the HIP paged KV cache.

``HipPagedAttention`` / ``HipPagedBlock`` stand next to the reference's
``FlashInferAttention`` / ``FlashInferBlock`` and ``SDPAAttention`` / ``SDPABlock``
(lingbot_map/layers/attention.py:352-556, lingbot_map/layers/block.py:151-310, :461-532):
same constructor arguments, same sub-module names (``norm1``, ``attn.qkv``, ``attn.q_norm``,
``attn.k_norm``, ``attn.proj``, ``ls1``, ``norm2``, ``mlp.fc1``, ``mlp.fc2``, ``ls2``) so a
reference state dict loads, the same ``forward`` signature, and the ``attn_pre`` /
``ffn_residual`` / ``attn.proj`` / ``attn.kv_cache_*`` attributes the reference's
compile recipe reaches into (gct_profile.py:51-56).

Differences, all inside the streaming branch:

* a keyframe's append, eviction and visible-row table are one index-kernel launch
  (``manager.step``) instead of three host-side list updates plus table uploads;
* a non-keyframe attends to the cache plus its own K/V read directly from the projection
  output; the reference appends, attends and rolls back (block.py:257-263), which writes
  8 MB per layer that no later frame reads.

Any manager with the reference call surface works: when ``kv_cache`` lacks ``step`` the
reference's method-by-method sequence is used.
"""
from __future__ import annotations

import math
import os
from typing import Callable, Optional

import torch
import torch.nn.functional as F
from torch import Tensor, nn


def apply_rotary_emb(x: Tensor, freqs: Tensor) -> Tensor:
    """Rotate interleaved (even, odd) pairs of ``x`` ``[B, H, N, D]`` by the complex
    ``freqs`` ``[1, 1, N, D/2]`` (lingbot_map/layers/rope.py:435-461)."""
    cos, sin = freqs.real.to(x.dtype), freqs.imag.to(x.dtype)
    x1, x2 = x[..., 0::2], x[..., 1::2]
    return torch.stack([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1).reshape(x.shape)


class RotaryPositionEmbedding2D(nn.Module):
    """2-D rotary embedding of the frame blocks (lingbot_map/layers/rope.py:64-198).

    The first half of head_dim belongs to the token's y coordinate and the second half to its
    x coordinate.  Inside a half of ``2q`` elements, element ``j < q`` and element ``j + q``
    form a pair that is turned by ``coordinate / frequency^(j / q)`` radians:
    ``(a, b) -> (a cos - b sin, b cos + a sin)``.  Everything is derived from one table,
    ``cos_sin_table``: a (cos, sin) per token and element, formed in the activations' dtype
    (angle, cosine and sine each rounded to it, as the reference's cached tables are) and
    handed to the fused producer as float32; ``forward`` is the same table applied with
    torch operations."""

    def __init__(self, frequency: float = 100.0, scaling_factor: float = 1.0) -> None:
        super().__init__()
        self.frequency = float(frequency)
        self.scaling_factor = float(scaling_factor)
        self._last_table = None

    def _pair_rates(self, pairs: int, device) -> Tensor:
        # radians per unit of coordinate for pair j of a half: the reciprocal of frequency^(j / pairs)
        j = torch.arange(pairs, device=device, dtype=torch.float32)
        return torch.reciprocal(torch.pow(self.frequency, (2.0 * j) / (2 * pairs)))

    def cos_sin_table(self, positions: Tensor, head_dim: int, dtype: torch.dtype) -> Tensor:
        """float32 ``[B * N, head_dim, 2]``: (cos, sin) of every element of every token for
        activations of ``dtype``; ``positions`` is ``[B, N, 2]`` integer (y, x).  The table of the
        last positions tensor is kept."""
        if positions.ndim != 3 or positions.shape[-1] != 2:
            raise ValueError(f"positions must be [batch, tokens, 2] (y, x), got {tuple(positions.shape)}")
        if head_dim % 4 != 0:
            raise ValueError(f"head_dim {head_dim} must split into two halves of pairs")
        key = (positions.data_ptr(), tuple(positions.shape), positions._version, head_dim, dtype)
        if self._last_table is not None and self._last_table[0] == key:
            return self._last_table[1]
        batch, n_tok, pairs = positions.shape[0], positions.shape[1], head_dim // 4
        # [B, N, axis, pair]: one float32 product per entry, then the activations' precision
        turn = (positions.to(torch.float32)[..., None] * self._pair_rates(pairs, positions.device)).to(dtype)
        # both members of a pair see the same angle: [B, N, axis, member, pair] = head_dim elements
        turn = turn[:, :, :, None, :].expand(batch, n_tok, 2, 2, pairs)
        table = torch.stack((torch.cos(turn), torch.sin(turn)), dim=-1).float().reshape(batch * n_tok, head_dim, 2)
        table = table.contiguous()
        self._last_table = (key, table, positions)   # the tensor stays alive with its key
        return table

    def forward(self, tokens: Tensor, positions: Tensor) -> Tensor:
        """``tokens`` ``[B, H, N, D]``, ``positions`` ``[B, N, 2]``; every product and the sum are
        rounded to the tokens' dtype."""
        batch, _, n_tok, dim = tokens.shape
        cs = self.cos_sin_table(positions, dim, tokens.dtype).view(batch, 1, n_tok, dim, 2).to(tokens.dtype)
        halves = tokens.reshape(*tokens.shape[:-1], 2, 2, dim // 4)          # [..., axis, member, pair]
        partner = torch.stack((-halves[..., 1, :], halves[..., 0, :]), dim=-2).reshape(tokens.shape)
        return tokens * cs[..., 0] + partner * cs[..., 1]


class PositionGetter:
    """(y, x) grid coordinates of a frame's patches, ``[B, height * width, 2]`` int64, row-major
    (lingbot_map/layers/rope.py:26-61).  One grid per (height, width, device) is kept."""

    def __init__(self) -> None:
        self.position_cache = {}

    def __call__(self, batch_size: int, height: int, width: int, device) -> Tensor:
        key = (height, width, torch.device(device))
        if key not in self.position_cache:
            idx = torch.arange(height * width, device=device)
            self.position_cache[key] = torch.stack((idx // width, idx % width), dim=-1)
        return self.position_cache[key].view(1, height * width, 2).expand(batch_size, -1, -1).clone()


class RotaryPositionEmbedding3D(nn.Module):
    """Complex rotary table of the global blocks (the reference's ``WanRotaryPosEmbed``,
    lingbot_map/layers/rope.py:279-432): the ``head_dim / 2`` interleaved pairs are dealt to
    the frame, row and column axes (10 / 11 / 11 pairs for head_dim 64) and pair j of an axis
    that owns ``dim`` elements rotates by ``coordinate * theta^(-2j/dim)``.  Special token i of
    frame f sits at (f, i, i); patch (y, x) at (f, n_special + y, n_special + x), or at
    (f, y, x) when there are no special tokens.  Frames count from ``f_start``.

    The reference precomputes ``exp(i * pos * freq)`` for every position below ``max_seq_len``
    and assembles a frame's table by slicing, expanding and concatenating; here each token's
    three integer coordinates are written down and the angles are one float64 product, which
    gives the same complex128 values and has no table to keep on the device."""

    def __init__(self, attention_head_dim: int, patch_size=(1, 14, 14), max_seq_len: int = 1024,
                 theta: float = 10000.0, fhw_dim=(20, 22, 22)) -> None:
        super().__init__()
        self.attention_head_dim = attention_head_dim
        self.patch_size = patch_size
        self.max_seq_len = max_seq_len
        self.theta = theta
        if fhw_dim is not None:
            assert attention_head_dim == sum(fhw_dim), \
                f"attention_head_dim {attention_head_dim} must match sum(fhw_dim) {sum(fhw_dim)}"
            t_dim, h_dim, w_dim = fhw_dim
        else:
            h_dim = w_dim = 2 * (attention_head_dim // 6)
            t_dim = attention_head_dim - h_dim - w_dim
        assert t_dim % 2 == 0 and h_dim % 2 == 0 and w_dim % 2 == 0, "every axis owns whole pairs"
        self.fhw_dim = (t_dim, h_dim, w_dim)
        inv_freq, axis = [], []
        for a, dim in enumerate(self.fhw_dim):
            inv_freq.append(1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim)))
            axis.append(torch.full((dim // 2,), a, dtype=torch.int64))
        self.register_buffer("inv_freq", torch.cat(inv_freq), persistent=False)   # [D/2] float64
        self.register_buffer("pair_axis", torch.cat(axis), persistent=False)      # [D/2] in {0, 1, 2}

    def coordinates(self, ppf: int, pph: int, ppw: int, patch_start_idx: int, device,
                    f_start: int = 0, f_end: Optional[int] = None) -> Tensor:
        """int64 ``[frames * (patch_start_idx + pph * ppw), 3]``: (frame, row, column) per token,
        specials first within each frame."""
        if f_end is not None:
            ppf = f_end - f_start
        else:
            f_start = 0
        assert 0 <= f_start and f_start + ppf <= self.max_seq_len, \
            f"frames [{f_start}, {f_start + ppf}) outside the {self.max_seq_len} positions of the table"
        assert patch_start_idx + max(pph, ppw) <= self.max_seq_len
        special = torch.arange(patch_start_idx, device=device)
        grid = torch.arange(pph * ppw, device=device)
        row = torch.cat((special, patch_start_idx + grid // ppw))
        col = torch.cat((special, patch_start_idx + grid % ppw))
        frame = torch.arange(f_start, f_start + ppf, device=device)
        n = row.numel()
        return torch.stack((frame[:, None].expand(ppf, n), row[None].expand(ppf, n), col[None].expand(ppf, n)),
                           dim=-1).reshape(ppf * n, 3)

    def angles(self, coords: Tensor) -> Tensor:
        """float64 ``[N, D/2]`` rotation angle of every pair."""
        inv_freq = self.inv_freq.to(coords.device)
        return coords.to(torch.float64)[:, self.pair_axis.to(coords.device)] * inv_freq

    def forward(self, ppf: int, pph: int, ppw: int, patch_start_idx: int, device,
                f_start: int = 0, f_end: Optional[int] = None) -> Tensor:
        """complex128 ``[1, 1, N, D/2]``, the argument ``pos`` of a global block with
        ``enable_3d_rope=True``."""
        ang = self.angles(self.coordinates(ppf, pph, ppw, patch_start_idx, device, f_start, f_end))
        return torch.polar(torch.ones_like(ang), ang)[None, None]


WanRotaryPosEmbed = RotaryPositionEmbedding3D   # the reference's name for it


class LayerScale(nn.Module):
    """lingbot_map/layers/layer_scale.py"""

    def __init__(self, dim: int, init_values: float = 1e-5) -> None:
        super().__init__()
        self.gamma = nn.Parameter(init_values * torch.ones(dim))

    def forward(self, x: Tensor) -> Tensor:
        return x * self.gamma


_split_workspaces = {}


def _prefetch_hint(t: Optional[Tensor]) -> None:
    """Tell the next GEMM launch of the package which memory the launch AFTER it will read
    (``lbm_linear_prefetch_hint``): the weights of the layer that follows, which would otherwise
    come from HBM when that layer starts - a frame walks through far more weight bytes than the
    caches hold.  The blocks' chain names, in front of each of its GEMMs, the weights of the one
    after it: proj's in front of the qkv projection, fc1's in front of proj, fc2's in front of fc1,
    and in front of fc2 the qkv projection's of the block that follows - while a frame is being
    captured into a HIP graph, where the GPU sets the pace; an eager frame is bound by the host's
    launches and is spared the four extra calls per block."""
    if t is None or not t.is_cuda:
        return
    import ctypes as C
    from . import _native as N
    N.lib.lbm_linear_prefetch_hint(C.c_void_p(t.data_ptr()), t.numel() * t.element_size())


def _split_workspace(device, nbytes: int) -> Optional[Tensor]:
    """Zero-filled device memory for launches that split K (``lbm_linear_norm``'s workspace; the
    launches leave its counters at zero), one per device and scratch lane; None when nothing is
    needed.  The blocks' launches of one lane on one device are serialised (one manager, one
    stream at a time), so they share it; a chain that may overlap them runs under
    ``_native.scratch_lane``.  It is never allocated or filled under stream capture: a graph would
    own the memory and replay the fill."""
    if nbytes <= 0:
        return None
    from . import _native as N
    lane = (device, N.current_scratch_lane())
    ws = _split_workspaces.get(lane)
    if ws is None or ws.numel() < nbytes:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("the K-split workspace must exist before a frame is captured: run the frame once "
                               "eagerly first (GraphedFrame does)")
        ws = _split_workspaces[lane] = torch.zeros(nbytes, dtype=torch.uint8, device=device)
    return ws


class RowStats:
    """What a block hands the next one in place of ``norm1(x)``: per row of ``x`` and column tile of
    the launch that wrote it, the mean and the sum of squared deviations (``lbm_linear_norm``'s
    ``out_stats``).  The consumer folds its LayerNorm into its linear layer (``FoldedNorm``) and
    reads ``x`` itself."""

    def __init__(self, stats: Tensor, tiles: int) -> None:
        self.stats, self.tiles = stats, tiles


class FoldedNorm:
    """A LayerNorm folded into the linear layer behind it: ``linear(norm(x))`` =
    ``rstd * (x @ w^T - mean * colsum) + bias`` with ``w = W * g`` (bf16), ``colsum`` its row sums
    and ``bias = B + W @ c`` for the LayerNorm's weight ``g`` and bias ``c``.  Kept per (norm,
    linear) pair until one of the four parameters changes."""

    @staticmethod
    def possible(norm, linear: nn.Linear) -> bool:
        return (type(norm) is nn.LayerNorm and norm.elementwise_affine and norm.bias is not None
                and tuple(norm.normalized_shape) == (linear.in_features,) and linear.weight.dtype == torch.bfloat16
                and linear.weight.is_cuda and linear.in_features % 128 == 0 and linear.out_features % 64 == 0)

    @staticmethod
    def of(owner: nn.Module, norm: nn.LayerNorm, linear: nn.Linear):
        """(weight bf16 [N, K], colsum float32 [N], bias float32 [N])"""
        ts = [norm.weight, norm.bias, linear.weight] + ([linear.bias] if linear.bias is not None else [])
        key = tuple((t._version, t.data_ptr(), t.device) for t in ts)
        cache = owner.__dict__.setdefault("_folded_norms", {})
        hit = cache.get((id(norm), id(linear)))
        if hit is None or hit[0] != key:
            with torch.no_grad():
                W = linear.weight.detach().float()
                w = (W * norm.weight.detach().float()[None, :]).to(torch.bfloat16).contiguous()
                bias = W @ norm.bias.detach().float()
                if linear.bias is not None:
                    bias = bias + linear.bias.detach().float()
                hit = cache[(id(norm), id(linear))] = (key, (w, w.float().sum(dim=1).contiguous(), bias.contiguous()))
        return hit[1]


class Mlp(nn.Module):
    """lingbot_map/layers/mlp.py (dropout omitted: inference only)"""

    def __init__(self, in_features: int, hidden_features: Optional[int] = None, act_layer=nn.GELU,
                 drop: float = 0.0, bias: bool = True) -> None:
        super().__init__()
        hidden_features = hidden_features or in_features
        self.fc1 = nn.Linear(in_features, hidden_features, bias=bias)
        self.act = act_layer()
        self.fc2 = nn.Linear(hidden_features, in_features, bias=bias)

    #: rows up to which the fused launches are used: one frame's rows run on 128 x 128 tiles, several
    #: streams' rows on 256 x 256 tiles where the launch has the columns for them (qkv, fc1)
    FUSED_MAX_ROWS = 1 << 16

    def _can_fuse_fc1(self, x: Tensor) -> bool:
        fc1 = self.fc1
        return (x.is_cuda and x.dtype == torch.bfloat16 and fc1.weight.dtype == torch.bfloat16
                and isinstance(self.act, nn.GELU) and self.act.approximate == "none"
                and fc1.in_features % 128 == 0 and fc1.out_features % 64 == 0
                and x.numel() // fc1.in_features <= self.FUSED_MAX_ROWS
                and not (torch.is_grad_enabled() and (x.requires_grad or fc1.weight.requires_grad)))

    def _bias_f32(self, m: nn.Linear) -> Optional[Tensor]:
        if m.bias is None:
            return None
        key = (m.bias._version, m.bias.data_ptr(), m.bias.device)
        cache = self.__dict__.setdefault("_bias_cache", {})
        if cache.get(id(m), (None,))[0] != key:
            cache[id(m)] = (key, m.bias.detach().float().contiguous())
        return cache[id(m)][1]

    def fc1_gelu(self, x: Tensor, norm: Optional[nn.LayerNorm] = None, stats: Optional[RowStats] = None) -> Tensor:
        """``act(fc1(x))`` as one kernel: the GEMM with bias and the exact GELU in its store
        (mlp.py:35-36), roundings as the two separate bf16 torch ops.  With ``norm`` and ``stats``:
        ``act(fc1(norm(x)))``, the LayerNorm folded into the launch (block.py:194-195)."""
        import ctypes as C
        from . import _native as N
        fc1 = self.fc1
        a = x.reshape(-1, fc1.in_features).contiguous()
        out = torch.empty(a.shape[0], fc1.out_features, dtype=x.dtype, device=x.device)
        p = lambda t: None if t is None else C.c_void_p(t.data_ptr())
        if norm is None:
            w = fc1.weight if fc1.weight.is_contiguous() else fc1.weight.contiguous()
            bias, row_norm = self._bias_f32(fc1), None
        else:
            w, colsum, bias = FoldedNorm.of(self, norm, fc1)
            row_norm = N.RowNorm(stats.stats.data_ptr(), colsum.data_ptr(), stats.tiles, float(norm.eps))
        N.check(N.lib.lbm_linear_norm(p(a), row_norm, p(w), p(bias), None, None, p(out), None, a.shape[0], fc1.out_features,
                                      fc1.in_features, N.LINEAR_BIAS_GELU, None, 0, N.stream_ptr(x.device)))
        return out.reshape(*x.shape[:-1], fc1.out_features)

    def forward(self, x: Tensor) -> Tensor:
        if self._can_fuse_fc1(x):
            return self.fc2(self.fc1_gelu(x))
        return self.fc2(self.act(self.fc1(x)))


class HipPagedAttention(nn.Module):
    def __init__(self, dim: int, num_heads: int = 8, qkv_bias: bool = True, proj_bias: bool = True,
                 attn_drop: float = 0.0, proj_drop: float = 0.0, norm_layer: Callable[..., nn.Module] = nn.LayerNorm,
                 qk_norm: bool = False, fused_attn: bool = True, rope=None,
                 kv_cache_sliding_window: int = 64, kv_cache_scale_frames: int = 8,
                 kv_cache_cross_frame_special: bool = True, kv_cache_include_scale_frames: bool = True,
                 kv_cache_camera_only: bool = False) -> None:
        super().__init__()
        assert dim % num_heads == 0, "dim should be divisible by num_heads"
        self.num_heads = num_heads
        self.head_dim = dim // num_heads
        self.qkv = nn.Linear(dim, dim * 3, bias=qkv_bias)
        self.q_norm = norm_layer(self.head_dim) if qk_norm else nn.Identity()
        self.k_norm = norm_layer(self.head_dim) if qk_norm else nn.Identity()
        self.proj = nn.Linear(dim, dim, bias=proj_bias)
        self.rope = rope
        self.kv_cache_sliding_window = kv_cache_sliding_window
        self.kv_cache_scale_frames = kv_cache_scale_frames
        self.kv_cache_cross_frame_special = kv_cache_cross_frame_special
        self.kv_cache_include_scale_frames = kv_cache_include_scale_frames
        self.kv_cache_camera_only = kv_cache_camera_only

    # ------------------------------------------------------------------ projections
    def _qkv(self, x: Tensor, pos, enable_3d_rope: bool):
        B, N, _ = x.shape
        qkv = self.qkv(x).reshape(B, N, 3, self.num_heads, self.head_dim).permute(2, 0, 3, 1, 4)
        q, k, v = qkv.unbind(0)  # each [B, H, N, D]
        q, k = self.q_norm(q), self.k_norm(k)
        if self.rope is not None and not enable_3d_rope:
            q, k = self.rope(q, pos), self.rope(k, pos)
        elif self.rope is not None:
            q, k = apply_rotary_emb(q, pos), apply_rotary_emb(k, pos)
        return q, k, v

    def prepare_qkv(self, x: Tensor, pos=None, enable_3d_rope: bool = False):
        """q, k, v of the streamed frame(s) as ``[B * tokens, H, D]``, specials first within
        each frame (attention.py:402-426; the reference squeezes a batch of one, here the
        batch axis carries the independent streams of a ragged batch)."""
        q, k, v = self._qkv(x, pos, enable_3d_rope)
        B, H, N, D = q.shape
        nhd = lambda t: t.permute(0, 2, 1, 3).reshape(B * N, H, D).contiguous()
        return nhd(q), nhd(k), nhd(v)

    # ------------------------------------------------------------------ cache traffic
    def _evict_kwargs(self, num_register_tokens: int) -> dict:
        return dict(scale_frames=self.kv_cache_scale_frames, sliding_window=self.kv_cache_sliding_window,
                    cross_frame_special=self.kv_cache_cross_frame_special,
                    include_scale_frames=self.kv_cache_include_scale_frames,
                    camera_only=self.kv_cache_camera_only, num_register_tokens=num_register_tokens)

    def stream_attend(self, manager, global_idx: int, q: Tensor, k: Tensor, v: Tensor,
                      num_register_tokens: int = 4) -> Tensor:
        """One streamed frame through the cache: block.py:256-278."""
        skip_append = getattr(manager, "_skip_append", False)
        if hasattr(manager, "step"):
            return manager.step(global_idx, q, k, v, keyframe=None,  # None: follows manager._skip_append
                                cross_frame_special=self.kv_cache_cross_frame_special,
                                camera_only=self.kv_cache_camera_only)
        if skip_append:
            prev = manager._defer_eviction
            manager._defer_eviction = True
            manager.append_frame(global_idx, k, v)
            out = manager.compute_attention(global_idx, q)
            manager.rollback_last_frame(global_idx)
            manager._defer_eviction = prev
            return out
        manager.append_frame(global_idx, k, v)
        manager.evict_frames(block_idx=global_idx, **self._evict_kwargs(num_register_tokens))
        return manager.compute_attention(global_idx, q)

    # ------------------------------------------------------------------ fused producer
    def can_fuse(self, manager, pos, enable_3d_rope: bool) -> bool:
        """Whether the manager's fused producer covers this module's pre-attention ops: plain
        LayerNorm (or none) on q and k and either no rotary embedding or the interleaved-pair
        one driven by a complex table (the 2-D variant of the frame blocks is not covered)."""
        if not hasattr(manager, "step_qkv") or self.head_dim != 64:
            return False
        norms = (self.q_norm, self.k_norm)
        if not (all(isinstance(m, nn.Identity) for m in norms) or
                all(type(m) is nn.LayerNorm and m.elementwise_affine and m.bias is not None for m in norms)):
            return False
        if self.rope is None:
            return True
        return bool(enable_3d_rope) and torch.is_tensor(pos) and pos.is_complex()

    def _norm_f32(self, m: nn.LayerNorm):
        key = (m.weight._version, m.bias._version, m.weight.data_ptr(), m.weight.device)
        cache = self.__dict__.setdefault("_norm_cache", {})
        if cache.get(id(m), (None,))[0] != key:
            cache[id(m)] = (key, (m.weight.detach().float().contiguous(), m.bias.detach().float().contiguous()))
        return cache[id(m)][1]

    def stream_attend_fused(self, manager, global_idx: int, x: Tensor, pos=None, norm=None, stats=None) -> Tensor:
        """qkv projection, then one kernel for q/k LayerNorm + rotary embedding + layout +
        paged append, then the paged attention (attention.py:402-426 and block.py:256-278).
        ``norm``, ``stats``: ``x`` is the block's input and ``norm`` is folded into the projection."""
        B, N, _ = x.shape
        proj = self._fused_projection(x, manager.dtype, norm, stats)
        qkv = None if proj is not None else self.qkv(x).reshape(B * N, -1)
        has_norm = isinstance(self.q_norm, nn.LayerNorm)
        rope_cs = None
        if self.rope is not None:
            rope_cs = torch.view_as_real(pos.to(torch.complex64)).reshape(-1, self.head_dim // 2, 2)
            assert rope_cs.shape[0] == N, f"rotary table for {rope_cs.shape[0]} tokens, frame has {N}"
            if B > 1:
                rope_cs = rope_cs.unsqueeze(0).expand(B, -1, -1, -1).reshape(B * N, self.head_dim // 2, 2)
        return manager.step_qkv(global_idx, qkv, self._norm_f32(self.q_norm) if has_norm else None,
                                self._norm_f32(self.k_norm) if has_norm else None, rope_cs,
                                norm_eps=self.q_norm.eps if has_norm else 1e-5, keyframe=None,
                                cross_frame_special=self.kv_cache_cross_frame_special,
                                camera_only=self.kv_cache_camera_only, proj=proj)

    #: rows up to which the projection with the producer as its epilogue is used (see Mlp.FUSED_MAX_ROWS)
    FUSED_PROJ_MAX_ROWS = 1 << 16

    def _fused_projection(self, x: Tensor, cache_dtype, norm: Optional[nn.LayerNorm] = None,
                          stats: Optional[RowStats] = None) -> Optional[tuple]:
        """(x [rows, K], weight, float32 bias) for ``lbm_qkv_linear_prepare`` when the projection
        can run in the producer's kernel: bf16 activations, weights and cache, head_dim 64, K a
        multiple of 128, one frame's worth of rows; None otherwise (the caller projects first).
        With ``norm`` and ``stats`` (``x`` is then the block's input, not ``norm(x)``) a fourth
        element: the ``lbm_row_norm`` of ``lbm_qkv_linear_prepare_norm``, weight and bias folded."""
        if norm is not None:
            from . import _native as N
            rows = x.numel() // x.shape[-1]
            w, colsum, bias = FoldedNorm.of(self, norm, self.qkv)
            norm.__dict__["_lbm_folded_qkv_weight"] = w    # where the block before this one finds it (_prefetch_hint)
            row_norm = N.RowNorm(stats.stats.data_ptr(), colsum.data_ptr(), stats.tiles, float(norm.eps))
            return x.reshape(rows, x.shape[-1]).contiguous(), w, bias, row_norm, (stats, colsum)
        w = self.qkv.weight
        rows = x.numel() // x.shape[-1]
        if not (x.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and cache_dtype == torch.bfloat16
                and self.head_dim == 64 and x.shape[-1] % 128 == 0 and rows <= self.FUSED_PROJ_MAX_ROWS
                and not (torch.is_grad_enabled() and (x.requires_grad or w.requires_grad))):
            return None
        bias = None
        if self.qkv.bias is not None:
            b = self.qkv.bias
            key = (b._version, b.data_ptr(), b.device)
            hit = self.__dict__.get("_qkv_bias_f32")
            if hit is None or hit[0] != key:
                hit = self.__dict__["_qkv_bias_f32"] = (key, b.detach().float().contiguous())
            bias = hit[1]
        return x.reshape(rows, x.shape[-1]).contiguous(), (w if w.is_contiguous() else w.contiguous()), bias

    def can_fold_norm(self, x: Tensor, norm, cache_dtype) -> bool:
        """Whether ``norm`` (the block's ``norm1``) can be folded into the fused projection."""
        rows = x.numel() // x.shape[-1]
        return (FoldedNorm.possible(norm, self.qkv) and x.is_cuda and x.dtype == torch.bfloat16
                and cache_dtype == torch.bfloat16 and self.head_dim == 64 and rows <= self.FUSED_PROJ_MAX_ROWS
                and not torch.is_grad_enabled())

    def can_fuse_dense(self, x: Tensor, pos, enable_3d_rope: bool) -> bool:
        """Whether the cache-less attention of a batch of frames can run as fused producer +
        paged kernel: GPU tensors, head_dim 64, plain LayerNorm or none on q and k, and no rotary
        embedding, the interleaved one with a complex table, or this package's 2-D one."""
        from . import _native as N
        if not (x.is_cuda and self.head_dim == 64 and x.dtype in (torch.bfloat16, torch.float32)):
            return False
        if not 1 <= x.shape[0] <= N.MAX_STREAMS:
            return False
        norms = (self.q_norm, self.k_norm)
        if not (all(isinstance(m, nn.Identity) for m in norms) or
                all(type(m) is nn.LayerNorm and m.elementwise_affine and m.bias is not None for m in norms)):
            return False
        if self.rope is None:
            return True
        if enable_3d_rope:
            return torch.is_tensor(pos) and pos.is_complex()
        return isinstance(self.rope, RotaryPositionEmbedding2D) and torch.is_tensor(pos) and pos.shape[0] in (1, x.shape[0])

    def dense_attend_fused(self, x: Tensor, pos=None, enable_3d_rope: bool = False, norm=None, stats=None,
                           return_kv: bool = False):
        """Attention of every frame of the batch over its own tokens (attention.py:446-465):
        qkv projection, one producer kernel, the paged kernel over a trivial row table.
        ``norm``, ``stats``: ``x`` is the block's input and ``norm`` is folded into the projection.
        ``return_kv``: also return k and v as ``[B * n, H, D]`` (after q/k norm and rotary
        embedding), which the anchor pass appends to the cache."""
        import ctypes as C
        from . import _native as N
        from .dense import dense_attention
        B, n, _ = x.shape
        H, D = self.num_heads, self.head_dim
        proj = self._fused_projection(x, x.dtype, norm, stats)
        qkv = None if proj is not None else self.qkv(x).reshape(B * n, -1).contiguous()
        has_norm = isinstance(self.q_norm, nn.LayerNorm)
        qk_norm = (self._norm_f32(self.q_norm) + self._norm_f32(self.k_norm)) if has_norm else (None,) * 4
        table, layout = None, N.ROPE_INTERLEAVED
        if self.rope is not None and enable_3d_rope:
            table = torch.view_as_real(pos.to(torch.complex64)).reshape(-1, D // 2, 2)
            if B > 1:
                table = table.unsqueeze(0).expand(B, -1, -1, -1).reshape(B * n, D // 2, 2)
            table = table.contiguous()
        elif self.rope is not None:
            positions = pos if pos.shape[0] == B else pos.expand(B, -1, -1)
            table, layout = self.rope.cos_sin_table(positions, D, x.dtype), N.ROPE_HALF_SPLIT
        if table is not None:
            assert table.shape[0] == B * n and table.dtype == torch.float32
        q, k, v = (torch.empty(B * n, H, D, dtype=x.dtype, device=x.device) for _ in range(3))
        p = lambda t: None if t is None else C.c_void_p(t.data_ptr())
        dt = N.DTYPE_BF16 if x.dtype == torch.bfloat16 else N.DTYPE_F32
        eps = float(self.q_norm.eps) if has_norm else 1e-5
        stream = N.stream_ptr(x.device)
        # q comes out multiplied by the softmax scale and log2(e) (rounded once), see dense_attention
        q_scale = N.q_scale_log2(1.0 / math.sqrt(D))
        if proj is not None:
            N.check(N.lib.lbm_qkv_linear_prepare_norm(
                p(proj[0]), proj[3] if len(proj) > 3 else None, p(proj[1]), p(proj[2]), B * n, proj[0].shape[1],
                p(qk_norm[0]), p(qk_norm[1]), p(qk_norm[2]), p(qk_norm[3]),
                eps, q_scale, p(table), layout, p(q), p(k), p(v), None, None, H, D, 16, stream))
        else:
            N.check(N.lib.lbm_qkv_prepare(
                p(qkv), dt, p(qk_norm[0]), p(qk_norm[1]), p(qk_norm[2]), p(qk_norm[3]), eps, q_scale, p(table), layout, p(q), p(k), p(v), dt,
                None, None, B * n, H, D, 16, stream))
        out = dense_attention(q, k, v, num_streams=B, q_prescaled=True).reshape(B, n, H * D)
        return (out, k, v) if return_kv else out

    def forward(self, x: Tensor, pos=None, num_patches=None, num_special=None, num_frames=None,
                enable_3d_rope=False, kv_cache=None, global_idx=0, num_frame_per_block=1,
                num_frame_for_scale=-1, num_register_tokens=4) -> Tensor:
        B, N, _ = x.shape
        has_manager = kv_cache is not None and hasattr(kv_cache, "append_frame")
        if not has_manager:
            # batch mode (attention.py:446-465)
            if self.can_fuse_dense(x, pos, enable_3d_rope):
                out = self.dense_attend_fused(x, pos, enable_3d_rope)
            else:
                q, k, v = self._qkv(x, pos, enable_3d_rope)
                out = F.scaled_dot_product_attention(q, k, v).transpose(1, 2).reshape(B, N, -1)
        elif num_frames is not None and num_frames > 1:
            # anchor pass over several frames: dense attention among them, then one append
            # and eviction per frame (attention.py:475-511).  Every stream of the batch attends
            # among its own frames; the cache takes the streams' frames side by side.
            tpf = kv_cache.tokens_per_frame
            assert N == num_frames * tpf, f"{N} tokens per stream are not {num_frames} frames of {tpf}"
            H, D = self.num_heads, self.head_dim
            if self.can_fuse_dense(x, pos, enable_3d_rope):
                # producer + the paged kernel over the streams' own rows (8 x 1005 rows per stream
                # at the reference's defaults: the split-KV kernel), no SDPA, no permutes
                out, k_all, v_all = self.dense_attend_fused(x, pos, enable_3d_rope, return_kv=True)
                k_all, v_all = k_all.view(B, num_frames, tpf, H, D), v_all.view(B, num_frames, tpf, H, D)
            else:
                q, k, v = self._qkv(x, pos, enable_3d_rope)
                out = F.scaled_dot_product_attention(q, k, v).transpose(1, 2).reshape(B, N, -1)
                k_all = k.permute(0, 2, 1, 3).reshape(B, num_frames, tpf, H, D)
                v_all = v.permute(0, 2, 1, 3).reshape(B, num_frames, tpf, H, D)
            for f in range(num_frames):
                kv_cache.append_frame(global_idx, k_all[:, f].reshape(B * tpf, H, D).contiguous(),
                                      v_all[:, f].reshape(B * tpf, H, D).contiguous())
                kv_cache.evict_frames(block_idx=global_idx, **self._evict_kwargs(num_register_tokens))
        else:
            if self.can_fuse(kv_cache, pos, enable_3d_rope):
                out = self.stream_attend_fused(kv_cache, global_idx, x, pos)
            else:
                q, k, v = self.prepare_qkv(x, pos=pos, enable_3d_rope=enable_3d_rope)
                out = self.stream_attend(kv_cache, global_idx, q, k, v, num_register_tokens)
            out = out.reshape(B, N, self.num_heads * self.head_dim).to(x.dtype)
        return self.proj(out)


class HipPagedBlock(nn.Module):
    #: name the next launch's weights in front of every GEMM of a captured frame (``_prefetch_hint``);
    #: a switch for measurements - results do not depend on it
    PREFETCH_HINTS = os.environ.get("LBM_PREFETCH_HINTS", "1") != "0"

    def __init__(self, dim: int, num_heads: int, mlp_ratio: float = 4.0, qkv_bias: bool = True,
                 proj_bias: bool = True, ffn_bias: bool = True, drop: float = 0.0, attn_drop: float = 0.0,
                 init_values=None, drop_path: float = 0.0, act_layer: Callable[..., nn.Module] = nn.GELU,
                 norm_layer: Callable[..., nn.Module] = nn.LayerNorm, ffn_layer: Callable[..., nn.Module] = Mlp,
                 qk_norm: bool = False, rope=None, kv_cache_sliding_window: int = 64,
                 kv_cache_scale_frames: int = 8, kv_cache_cross_frame_special: bool = True,
                 kv_cache_include_scale_frames: bool = True, kv_cache_camera_only: bool = False) -> None:
        super().__init__()
        self.norm1 = norm_layer(dim)
        self.attn = HipPagedAttention(
            dim=dim, num_heads=num_heads, qk_norm=qk_norm, qkv_bias=qkv_bias, proj_bias=proj_bias,
            attn_drop=attn_drop, proj_drop=drop, rope=rope,
            kv_cache_sliding_window=kv_cache_sliding_window, kv_cache_scale_frames=kv_cache_scale_frames,
            kv_cache_cross_frame_special=kv_cache_cross_frame_special,
            kv_cache_include_scale_frames=kv_cache_include_scale_frames,
            kv_cache_camera_only=kv_cache_camera_only)
        self.ls1 = LayerScale(dim, init_values=init_values) if init_values else nn.Identity()
        self.drop_path1 = nn.Identity()
        self.norm2 = norm_layer(dim)
        self.mlp = ffn_layer(in_features=dim, hidden_features=int(dim * mlp_ratio), act_layer=act_layer,
                             drop=drop, bias=ffn_bias)
        self.ls2 = LayerScale(dim, init_values=init_values) if init_values else nn.Identity()
        self.drop_path2 = nn.Identity()
        self.sample_drop_ratio = drop_path

    # ------------------------------------------------------------------ fused residual path
    def _f32(self, t: Tensor) -> Tensor:
        """float32 copy of a parameter, cached until the parameter changes."""
        cache = self.__dict__.setdefault("_f32_cache", {})
        key = (t._version, t.data_ptr(), t.device)
        hit = cache.get(id(t))
        if hit is None or hit[0] != key:
            cache[id(t)] = hit = (key, t.detach().float().contiguous())
        return hit[1]

    def _can_fuse_residual(self, x: Tensor) -> bool:
        return (x.is_cuda and x.dtype in (torch.bfloat16, torch.float32) and x.shape[-1] % 8 == 0
                and x.shape[-1] <= 8192 and type(self.norm2) is nn.LayerNorm and self.norm2.elementwise_affine
                and self.norm2.bias is not None and isinstance(self.ls1, (LayerScale, nn.Identity))
                and isinstance(self.ls2, (LayerScale, nn.Identity)) and not torch.is_grad_enabled())

    def _residual(self, x: Tensor, y: Tensor, ls, norm: Optional[nn.LayerNorm]):
        """x + ls(y) and, when ``norm`` is given, norm(x + ls(y)), in one kernel (block.py:283 and
        :194-195; layer_scale.py:21-22)."""
        import ctypes as C
        from . import _native as N
        x, y = x.contiguous(), y.contiguous().to(x.dtype)
        x_out = torch.empty_like(x)
        n_out = torch.empty_like(x) if norm is not None else None
        p = lambda t: None if t is None else C.c_void_p(t.data_ptr())
        gamma = self._f32(ls.gamma) if isinstance(ls, LayerScale) else None
        w, b = (self._f32(norm.weight), self._f32(norm.bias)) if norm is not None else (None, None)
        N.check(N.lib.lbm_residual_norm(
            p(x), p(y), N.DTYPE_BF16 if x.dtype == torch.bfloat16 else N.DTYPE_F32, p(gamma), p(w), p(b),
            float(norm.eps) if norm is not None else 0.0, p(x_out), p(n_out), x.numel() // x.shape[-1], x.shape[-1],
            N.stream_ptr(x.device)))
        return x_out, n_out

    def _finish(self, x: Tensor, attn_out: Tensor, next_norm: Optional[nn.LayerNorm] = None):
        """x + ls1(attn_out), then the MLP branch (block.py:283-285).  With ``next_norm`` (the
        ``norm1`` of the block that follows) returns ``(x, next_norm(x))``: the LayerNorm rides on
        the last residual kernel instead of being a launch of its own in the next block."""
        if self._can_fuse_residual(x):
            x, n = self._residual(x, attn_out, self.ls1, self.norm2)
            fuse_next = (next_norm is not None and type(next_norm) is nn.LayerNorm and next_norm.elementwise_affine
                         and next_norm.bias is not None)
            x, n_next = self._residual(x, self.mlp(n), self.ls2, next_norm if fuse_next else None)
            if next_norm is None:
                return x
            return x, (n_next if fuse_next else next_norm(x))
        x = self.ffn_residual(x + self.ls1(attn_out))
        return x if next_norm is None else (x, next_norm(x))

    # ------------------------------------------------------------------ the block as a chain of fused launches
    def _can_chain(self, x: Tensor, kv_cache, pos, enable_3d_rope: bool, streaming: bool) -> bool:
        """Whether the block can run as: qkv projection (+ folded norm1) + producer, attention,
        proj + LayerScale + residual (+ row statistics), fc1 (+ folded norm2) + GELU, fc2 +
        LayerScale + residual (+ row statistics) - five GEMM launches and the attention, no
        LayerNorm or residual kernel.  One frame's rows of bf16 on the GPU, inference."""
        a, rows = self.attn, x.numel() // x.shape[-1]
        if not (x.is_cuda and x.dtype == torch.bfloat16 and rows <= Mlp.FUSED_MAX_ROWS and not torch.is_grad_enabled()):
            return False
        if not (type(self.mlp) is Mlp and self.mlp._can_fuse_fc1(x) and FoldedNorm.possible(self.norm2, self.mlp.fc1)):
            return False
        if not all(isinstance(ls, (LayerScale, nn.Identity)) for ls in (self.ls1, self.ls2)):
            return False
        for lin in (a.proj, self.mlp.fc2):
            if not (lin.weight.dtype == torch.bfloat16 and lin.weight.is_cuda and lin.in_features % 128 == 0
                    and lin.out_features % 64 == 0):
                return False
        if streaming:
            return a.can_fuse(kv_cache, pos, enable_3d_rope) and kv_cache.dtype == torch.bfloat16
        return a.can_fuse_dense(x, pos, enable_3d_rope)

    def _linear_residual(self, a: Tensor, linear: nn.Linear, ls, residual: Tensor, want_stats: bool):
        """``residual + ls(linear(a))`` as one launch (attention.py:554 / mlp.py:38 with
        layer_scale.py:21-22 and block.py:283-285), and the row statistics of the result for the
        LayerNorm that reads it next."""
        import ctypes as C
        from . import _native as N
        rows, n_out = a.numel() // a.shape[-1], linear.out_features
        a2, res = a.reshape(rows, -1).contiguous(), residual.reshape(rows, n_out).contiguous()
        out = torch.empty_like(res)
        stats = None
        if want_stats:
            tiles = int(N.lib.lbm_linear_stats_tiles(rows, n_out))
            stats = RowStats(torch.empty(rows, tiles, 2, dtype=torch.float32, device=a.device), tiles)
        w = linear.weight if linear.weight.is_contiguous() else linear.weight.contiguous()
        bias = self._f32(linear.bias) if linear.bias is not None else None
        gamma = self._f32(ls.gamma) if isinstance(ls, LayerScale) else None
        p = lambda t: None if t is None else C.c_void_p(t.data_ptr())
        ws = _split_workspace(a.device, int(N.lib.lbm_linear_workspace_bytes(rows, n_out, a2.shape[1], N.LINEAR_BIAS_RESIDUAL)))
        N.check(N.lib.lbm_linear_norm(p(a2), None, p(w), p(bias), p(gamma), p(res), p(out),
                                      p(stats.stats) if stats is not None else None, rows, n_out, a2.shape[1],
                                      N.LINEAR_BIAS_RESIDUAL, p(ws), ws.numel() if ws is not None else 0,
                                      N.stream_ptr(a.device)))
        return out.reshape(residual.shape), stats

    def _finish_chain(self, x: Tensor, heads_out: Tensor, next_norm, hints: bool = False):
        """Everything after the attention kernel (block.py:283-285) in three launches;
        ``heads_out`` is the attention's output before ``proj``.  With ``next_norm`` the result is
        ``(x, RowStats)``: the statistics the next block folds its ``norm1`` from.  ``hints``: name
        the next launch's weights in front of each launch (``_prefetch_hint``)."""
        if hints:
            _prefetch_hint(FoldedNorm.of(self.mlp, self.norm2, self.mlp.fc1)[0])
        x, stats = self._linear_residual(heads_out, self.attn.proj, self.ls1, x, True)
        if hints:
            _prefetch_hint(self.mlp.fc2.weight)
        hidden = self.mlp.fc1_gelu(x, self.norm2, stats)
        if hints:
            _prefetch_hint(getattr(next_norm, "_lbm_folded_qkv_weight", None))
        x, stats = self._linear_residual(hidden, self.mlp.fc2, self.ls2, x, next_norm is not None)
        return x if next_norm is None else (x, stats)

    def attn_pre(self, x: Tensor, pos=None, enable_3d_rope: bool = False):
        """norm1 + projections + qk-norm + RoPE, ready for the cache (block.py:217-227)."""
        return self.attn.prepare_qkv(self.norm1(x), pos=pos, enable_3d_rope=enable_3d_rope)

    def ffn_residual(self, x: Tensor) -> Tensor:
        return x + self.ls2(self.mlp(self.norm2(x)))

    def forward(self, x: Tensor, pos=None, num_patches=None, num_special=None, num_frames=None,
                enable_3d_rope=False, kv_cache=None, global_idx=0, num_frame_per_block=1,
                num_frame_for_scale=-1, num_register_tokens=4, normed: Optional[Tensor] = None,
                next_norm: Optional[nn.LayerNorm] = None):
        """The reference's arguments (block.py:229-243) plus two for a caller that chains blocks:
        ``normed`` = ``self.norm1(x)`` if the caller already has it - or the ``RowStats`` of ``x``
        the block before left behind - and ``next_norm`` = the ``norm1`` of the block that follows;
        with ``next_norm`` the result is ``(x, next_norm(x))`` or ``(x, RowStats of x)``."""
        is_streaming = kv_cache is not None and (num_frames is None or num_frames <= 1)
        is_dense = kv_cache is None or not hasattr(kv_cache, "append_frame")
        stats = normed if isinstance(normed, RowStats) else None
        if (is_streaming or is_dense) and self._can_chain(x, kv_cache, pos, enable_3d_rope, is_streaming):
            cache_dtype = kv_cache.dtype if is_streaming else x.dtype
            fold = stats is not None and self.attn.can_fold_norm(x, self.norm1, cache_dtype)
            if fold:
                a_in, kw = x, dict(norm=self.norm1, stats=stats)
            else:
                a_in, kw = (self.norm1(x) if (normed is None or stats is not None) else normed), {}
            # (hints only where the GPU sets the pace: an eager frame is bound by the host's launches,
            # and four more calls per block would slow it)
            hints = self.PREFETCH_HINTS and torch.cuda.is_current_stream_capturing()
            if hints:
                _prefetch_hint(self.attn.proj.weight)
            if is_streaming:
                heads = self.attn.stream_attend_fused(kv_cache, global_idx, a_in, pos, **kw)
            else:
                heads = self.attn.dense_attend_fused(a_in, pos, enable_3d_rope, **kw)
            heads = heads.reshape(x.shape[0], x.shape[1], self.attn.num_heads * self.attn.head_dim).to(x.dtype)
            return self._finish_chain(x, heads, next_norm, hints)
        n1 = self.norm1(x) if (normed is None or stats is not None) else normed
        if is_streaming:
            if self.attn.can_fuse(kv_cache, pos, enable_3d_rope):
                attn_x = self.attn.stream_attend_fused(kv_cache, global_idx, n1, pos)
            else:
                q, k, v = self.attn.prepare_qkv(n1, pos=pos, enable_3d_rope=enable_3d_rope)
                attn_x = self.attn.stream_attend(kv_cache, global_idx, q, k, v, num_register_tokens)
            attn_x = attn_x.reshape(x.shape[0], x.shape[1], self.attn.num_heads * self.attn.head_dim).to(x.dtype)
            return self._finish(x, self.attn.proj(attn_x), next_norm)
        return self._finish(x, self.attn(
            n1, pos=pos, num_patches=num_patches, num_special=num_special, num_frames=num_frames,
            enable_3d_rope=enable_3d_rope, kv_cache=kv_cache, global_idx=global_idx,
            num_frame_per_block=num_frame_per_block, num_frame_for_scale=num_frame_for_scale,
            num_register_tokens=num_register_tokens), next_norm)


def keyframe_flags(num_frames: int, scale_frames: int, keyframe_interval: int):
    """Which streamed frames are cached (lingbot_map/models/gct_stream.py:450): the anchor
    frames always, afterwards every ``keyframe_interval``-th frame."""
    return [i < scale_frames or keyframe_interval <= 1 or (i - scale_frames) % keyframe_interval == 0
            for i in range(num_frames)]


def set_skip_append(manager, skip: bool) -> None:
    """The driver's non-keyframe switch (lingbot_map/models/gct_stream.py:300-318)."""
    manager._skip_append = bool(skip)
