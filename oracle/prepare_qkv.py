"""CPU oracle: the pre-attention producer of the reference's streaming path.

TEST INFRASTRUCTURE ONLY (see oracle/page_policy.py for who may import this package).

Restated from the reference (paths relative to its checkout):

* split of the qkv projection output into q, k, v of ``[B, H, N, D]``, per-head LayerNorm of
  q and k, rotary embedding, ``[N, H, D]`` contiguous copies
                                           lingbot_map/layers/attention.py:402-426
* rotary embedding on interleaved (even, odd) pairs with a complex table, cos and sin cast
  to the activations' dtype, plain elementwise arithmetic in that dtype
                                           lingbot_map/layers/rope.py:438-461

``prepare_qkv`` runs the same torch operations in the same order and dtype as the reference,
so for bf16 activations every intermediate is rounded where the reference rounds it
(LayerNorm output, cos, sin, each product, each sum).

Parity pins (tests/test_oracle_prepare.py): rotation by angle 0 is the identity, by 90
degrees maps (a, b) to (-b, a); in fp32 the result equals the complex product
``view_as_complex(x) * freqs`` and preserves the norm of every pair; LayerNorm of a
constant row is the bias and otherwise equals a float64 restatement of
(x - mean) / sqrt(var + eps) * w + b; v passes through unchanged; the layout is the
transpose the reference's permutes describe.
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


def prepare_qkv(qkv: torch.Tensor, num_heads: int, head_dim: int,
                q_norm: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                k_norm: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                freqs: Optional[torch.Tensor] = None, eps: float = 1e-5):
    """qkv ``[N, 3 * H * D]`` (one stream, batch of one) -> q, k, v of ``[N, H, D]``
    (attention.py:412-426).  ``q_norm`` / ``k_norm``: (weight, bias) in the activations' dtype."""
    n = qkv.shape[0]
    t = qkv.reshape(1, n, 3, num_heads, head_dim).permute(2, 0, 3, 1, 4)
    q, k, v = t.unbind(0)  # each [1, H, N, D]
    if q_norm is not None:
        q = F.layer_norm(q, (head_dim,), q_norm[0], q_norm[1], eps)
        k = F.layer_norm(k, (head_dim,), k_norm[0], k_norm[1], eps)
    if freqs is not None:
        q = apply_rotary_emb(q, freqs)
        k = apply_rotary_emb(k, freqs)
    nhd = lambda z: z.squeeze(0).permute(1, 0, 2).contiguous()
    return nhd(q), nhd(k), nhd(v)
