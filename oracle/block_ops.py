"""CPU oracle: the residual update of a block with the LayerNorm that follows it, and the
block's linear layers with the elementwise operations that follow them.

TEST INFRASTRUCTURE ONLY (see oracle/page_policy.py for who may import this package).

Restated from the reference (paths relative to its checkout):

* ``x = x + ls1(attn_out)`` and ``x + ls2(mlp(norm2(x)))``
                                           lingbot_map/layers/block.py:194-195,283
* LayerScale is an elementwise product with ``gamma``
                                           lingbot_map/layers/layer_scale.py:21-22
* norm2 is ``nn.LayerNorm(dim)``            lingbot_map/layers/block.py:203

* the linears: ``qkv`` (lingbot_map/layers/attention.py:413), ``proj`` (:554), ``fc1`` followed by the
  exact GELU and ``fc2`` (lingbot_map/layers/mlp.py:35-38)

``residual_norm`` runs the same torch operations in the same order and dtype.  ``linear_epilogue``
accumulates the product in fp32 on the CPU and then rounds where the separate bf16 torch
operations of the reference round: after the linear (bias added in fp32 first, as the library
GEMM's own epilogue does), after the GELU or the LayerScale product, after the residual add.

Parity pins (tests/test_oracle_prepare.py): gamma = 0 leaves x unchanged and gamma = 1 gives
x + y; a float64 restatement of x + y * gamma and of the LayerNorm definition; the LayerNorm of
a row whose update makes it constant is the bias.  ``linear_epilogue``: an identity weight returns
the input plus the bias; GELU(0) = 0, GELU(x) -> x for large x and -> 0 for very negative x, and
GELU(x) - GELU(-x) = x; gamma = 0 returns the residual; a float64 three-loop product on a tiny
shape (a transposed weight fails it).
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F


def residual_norm(x: torch.Tensor, y: torch.Tensor, gamma: Optional[torch.Tensor],
                  norm_w: Optional[torch.Tensor] = None, norm_b: Optional[torch.Tensor] = None, eps: float = 1e-5):
    """Returns (x + y * gamma, LayerNorm of that or None)."""
    x_new = x + (y * gamma if gamma is not None else y)
    n = F.layer_norm(x_new, (x.shape[-1],), norm_w, norm_b, eps) if norm_w is not None else None
    return x_new, n


LINEAR_BIAS, LINEAR_BIAS_GELU, LINEAR_BIAS_RESIDUAL = 0, 1, 2


def linear_epilogue(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], epilogue: int,
                    gamma: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``a`` [M, K], ``w`` [N, K] (nn.Linear's weight), bf16 values; returns float32 holding bf16 values."""
    bf = lambda t: t.to(torch.bfloat16).float()
    y = a.float() @ w.float().t()
    if bias is not None:
        y = y + bias.float()
    y = bf(y)
    if epilogue == LINEAR_BIAS_GELU:
        y = bf(F.gelu(y))
    if epilogue == LINEAR_BIAS_RESIDUAL:
        if gamma is not None:
            y = bf(y * gamma.float())
        y = bf(residual.float() + y)
    return y
