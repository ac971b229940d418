"""CPU oracle: the pre-attention producer of the reference's streaming path.

TEST INFRASTRUCTURE ONLY (see oracle/page_policy.py for who may import this package).

Restated from the reference (paths relative to its checkout):

* split of the qkv projection output into q, k, v of ``[B, H, N, D]``, per-head LayerNorm of
  q and k, rotary embedding, ``[N, H, D]`` contiguous copies
                                           lingbot_map/layers/attention.py:402-426
* rotary embedding on interleaved (even, odd) pairs with a complex table, cos and sin cast
  to the activations' dtype, plain elementwise arithmetic in that dtype
                                           lingbot_map/layers/rope.py:438-461

* 2-D rotary embedding of the frame blocks: head_dim split into a vertical and a horizontal
  half, each rotated as x * cos + rotate(x) * sin with rotate = (-second half, first half),
  angle table pos * base^(-2j/dim) repeated twice, computed and cast in the activations' dtype
                                           lingbot_map/layers/rope.py:86-198

* complex table of the global blocks' 3-D rotary embedding: one 1-D table
  exp(i * pos * theta^(-2j/dim)) per axis in float64, concatenated along the pair axis, then
  sliced per axis (frames f_start..f_end, rows and columns offset by the number of special
  tokens, special token i at row i and column i), expanded and concatenated per frame
                                           lingbot_map/layers/rope.py:202-276, :279-432

``prepare_qkv`` runs the same torch operations in the same order and dtype as the reference,
so for bf16 activations every intermediate is rounded where the reference rounds it
(LayerNorm output, cos, sin, each product, each sum).

Parity pins (tests/test_oracle_prepare.py): rotation by angle 0 is the identity, by 90
degrees maps (a, b) to (-b, a); in fp32 the result equals the complex product
``view_as_complex(x) * freqs`` and preserves the norm of every pair; LayerNorm of a
constant row is the bias and otherwise equals a float64 restatement of
(x - mean) / sqrt(var + eps) * w + b; v passes through unchanged; the layout is the
transpose the reference's permutes describe.  ``rope2d``: position (0, 0) is the identity; in
float64 element j of a half and element j + dim/4 rotate by pos * base^(-4j/dim) (an explicit
loop restates it), pair norms are kept, the vertical half ignores x and the horizontal half y.
``rope3d_freqs``: every entry has modulus 1; the entry of a named token and pair equals
exp(i * coordinate * theta^(-2j/dim)) written out by hand for the camera token, a register
token and two patches; shifting f_start changes the frame pairs only; frame 0 of a two-frame
table equals the one-frame table; without special tokens the patch grid starts at (0, 0).
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F


def apply_rotary_emb(x: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """x ``[B, H, N, D]``, freqs complex ``[1, 1, N, D/2]`` (rope.py:438-461)."""
    cos = freqs.real.to(x.dtype)
    sin = freqs.imag.to(x.dtype)
    x1 = x[..., 0::2]
    x2 = x[..., 1::2]
    out1 = x1 * cos - x2 * sin
    out2 = x1 * sin + x2 * cos
    return torch.stack([out1, out2], dim=-1).reshape(x.shape)


def rope2d_tables(dim: int, seq_len: int, dtype: torch.dtype, base: float = 100.0):
    """cos / sin tables ``[seq_len, dim]`` of one spatial direction (rope.py:86-122)."""
    exponents = torch.arange(0, dim, 2).float() / dim
    inv_freq = 1.0 / (base ** exponents)
    positions = torch.arange(seq_len, dtype=inv_freq.dtype)
    angles = torch.einsum("i,j->ij", positions, inv_freq)
    angles = angles.to(dtype)
    angles = torch.cat((angles, angles), dim=-1)
    return angles.cos().to(dtype), angles.sin().to(dtype)


def rope2d(tokens: torch.Tensor, positions: torch.Tensor, base: float = 100.0) -> torch.Tensor:
    """tokens ``[B, H, N, D]``, positions ``[B, N, 2]`` integer (y, x) (rope.py:154-198)."""
    feature_dim = tokens.size(-1) // 2
    cos_comp, sin_comp = rope2d_tables(feature_dim, positions.shape[1], tokens.dtype, base)

    def rotate(x):
        d = x.shape[-1]
        return torch.cat((-x[..., d // 2:], x[..., : d // 2]), dim=-1)

    def one(x, pos):
        cos = F.embedding(pos, cos_comp)[:, None, :, :]
        sin = F.embedding(pos, sin_comp)[:, None, :, :]
        return (x * cos) + (rotate(x) * sin)

    vert, horiz = tokens.chunk(2, dim=-1)
    return torch.cat((one(vert, positions[..., 0]), one(horiz, positions[..., 1])), dim=-1)


def rope3d_axis_table(dim: int, n_pos: int, theta: float = 10000.0) -> torch.Tensor:
    """complex128 ``[n_pos, dim / 2]`` of one axis (rope.py:202-276 with freqs_dtype float64)."""
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64)[: dim // 2] / dim))
    ang = torch.outer(torch.arange(n_pos), freqs)
    return torch.polar(torch.ones_like(ang), ang)


def rope3d_freqs(ppf: int, pph: int, ppw: int, patch_start_idx: int, head_dim: int = 64,
                 fhw_dim=(20, 22, 22), max_seq_len: int = 1024, theta: float = 10000.0,
                 f_start: int = 0, f_end: Optional[int] = None) -> torch.Tensor:
    """complex128 ``[1, 1, frames * (patch_start_idx + pph * ppw), head_dim / 2]``
    (rope.py:299-432)."""
    assert sum(fhw_dim) == head_dim
    tab_f, tab_h, tab_w = (rope3d_axis_table(d, max_seq_len, theta) for d in fhw_dim)
    if f_end is not None:
        ppf = f_end - f_start
        tab_f = tab_f[f_start:f_end]
    else:
        tab_f = tab_f[:ppf]
    s = patch_start_idx
    per_frame = []
    if s > 0:
        per_frame.append(torch.cat((tab_f.reshape(ppf, 1, -1).expand(ppf, s, -1),
                                    tab_h[:s].reshape(1, s, -1).expand(ppf, s, -1),
                                    tab_w[:s].reshape(1, s, -1).expand(ppf, s, -1)), dim=-1))
    patches = torch.cat((tab_f.reshape(ppf, 1, 1, -1).expand(ppf, pph, ppw, -1),
                         tab_h[s:s + pph].reshape(1, pph, 1, -1).expand(ppf, pph, ppw, -1),
                         tab_w[s:s + ppw].reshape(1, 1, ppw, -1).expand(ppf, pph, ppw, -1)), dim=-1)
    per_frame.append(patches.reshape(ppf, pph * ppw, -1))
    return torch.cat(per_frame, dim=1).reshape(1, 1, ppf * (s + pph * ppw), -1)


def prepare_qkv(qkv: torch.Tensor, num_heads: int, head_dim: int,
                q_norm: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                k_norm: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                freqs: Optional[torch.Tensor] = None, eps: float = 1e-5,
                positions: Optional[torch.Tensor] = None):
    """qkv ``[N, 3 * H * D]`` (one stream, batch of one) -> q, k, v of ``[N, H, D]``
    (attention.py:412-426).  ``q_norm`` / ``k_norm``: (weight, bias) in the activations' dtype.
    ``freqs``: complex table of the interleaved embedding (global blocks); ``positions``
    ``[N, 2]``: the 2-D embedding of the frame blocks instead."""
    n = qkv.shape[0]
    t = qkv.reshape(1, n, 3, num_heads, head_dim).permute(2, 0, 3, 1, 4)
    q, k, v = t.unbind(0)  # each [1, H, N, D]
    if q_norm is not None:
        q = F.layer_norm(q, (head_dim,), q_norm[0], q_norm[1], eps)
        k = F.layer_norm(k, (head_dim,), k_norm[0], k_norm[1], eps)
    if freqs is not None:
        q = apply_rotary_emb(q, freqs)
        k = apply_rotary_emb(k, freqs)
    elif positions is not None:
        q = rope2d(q, positions[None])
        k = rope2d(k, positions[None])
    nhd = lambda z: z.squeeze(0).permute(1, 0, 2).contiguous()
    return nhd(q), nhd(k), nhd(v)
