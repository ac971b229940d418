"""CPU oracle: the residual update of a block and the LayerNorm that follows it.

TEST INFRASTRUCTURE ONLY (see oracle/page_policy.py for who may import this package).

Restated from the reference (paths relative to its checkout):

* ``x = x + ls1(attn_out)`` and ``x + ls2(mlp(norm2(x)))``
                                           lingbot_map/layers/block.py:194-195,283
* LayerScale is an elementwise product with ``gamma``
                                           lingbot_map/layers/layer_scale.py:21-22
* norm2 is ``nn.LayerNorm(dim)``            lingbot_map/layers/block.py:203

``residual_norm`` runs the same torch operations in the same order and dtype.

Parity pins (tests/test_oracle_prepare.py): gamma = 0 leaves x unchanged and gamma = 1 gives
x + y; a float64 restatement of x + y * gamma and of the LayerNorm definition; the LayerNorm of
a row whose update makes it constant is the bias.
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
