"""Pins of oracle/prepare_qkv.py by what the mathematics fixes (no GPU)."""
import math

import torch

from oracle.prepare_qkv import apply_rotary_emb, prepare_qkv, rope2d


def _freqs(n, d, seed=0, angle=None):
    g = torch.Generator().manual_seed(seed)
    ang = torch.rand(1, 1, n, d // 2, generator=g) * 2 * math.pi if angle is None else torch.full((1, 1, n, d // 2), angle)
    return torch.polar(torch.ones_like(ang), ang)


def test_rotation_by_zero_and_by_a_quarter_turn():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 2, 5, 64, generator=g)
    assert torch.equal(apply_rotary_emb(x, _freqs(5, 64, angle=0.0)), x)
    quarter = torch.complex(torch.zeros(1, 1, 5, 32), torch.ones(1, 1, 5, 32))   # cos 0, sin 1 exactly
    y = apply_rotary_emb(x, quarter)
    assert torch.equal(y[..., 0::2], -x[..., 1::2]) and torch.equal(y[..., 1::2], x[..., 0::2])


def test_rotation_equals_the_complex_product_and_keeps_pair_norms():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, 3, 7, 64, generator=g, dtype=torch.float64)
    ang = torch.rand(1, 1, 7, 32, generator=g, dtype=torch.float64) * 2 * math.pi
    fr = torch.polar(torch.ones_like(ang), ang)
    y = apply_rotary_emb(x, fr)
    z = torch.view_as_real(torch.view_as_complex(x.reshape(1, 3, 7, 32, 2).contiguous()) * fr).reshape(x.shape)
    assert (y - z).abs().max().item() < 1e-14
    n_in = x.reshape(1, 3, 7, 32, 2).norm(dim=-1)
    n_out = y.reshape(1, 3, 7, 32, 2).norm(dim=-1)
    assert (n_in - n_out).abs().max().item() < 1e-13


def test_layernorm_closed_forms_and_float64_restatement():
    H, D, n = 2, 64, 6
    g = torch.Generator().manual_seed(4)
    w, b = torch.randn(D, generator=g), torch.randn(D, generator=g)
    const = torch.full((n, 3 * H * D), 1.75)
    q, k, v = prepare_qkv(const, H, D, (w, b), (w, b), None, eps=1e-5)
    assert torch.allclose(q, b.expand(n, H, D), atol=1e-6) and torch.allclose(k, b.expand(n, H, D), atol=1e-6)
    assert torch.equal(v, torch.full((n, H, D), 1.75))
    x = torch.randn(n, 3 * H * D, generator=g)
    q, k, v = prepare_qkv(x, H, D, (w, b), (2 * w, -b), None, eps=1e-5)
    x5 = x.double().reshape(n, 3, H, D)
    for which, got, ww, bb in ((0, q, w, b), (1, k, 2 * w, -b)):
        z = x5[:, which]
        mean = z.mean(-1, keepdim=True)
        var = ((z - mean) ** 2).mean(-1, keepdim=True)          # biased, as LayerNorm defines it
        want = (z - mean) / torch.sqrt(var + 1e-5) * ww.double() + bb.double()
        assert (got.double() - want).abs().max().item() < 1e-5
    assert torch.equal(v, x.reshape(n, 3, H, D)[:, 2])


def test_layout_is_token_head_dim_of_the_projection_output():
    H, D, n = 3, 64, 4
    x = torch.arange(n * 3 * H * D, dtype=torch.float32).reshape(n, 3 * H * D)
    q, k, v = prepare_qkv(x, H, D)
    x5 = x.reshape(n, 3, H, D)
    assert torch.equal(q, x5[:, 0]) and torch.equal(k, x5[:, 1]) and torch.equal(v, x5[:, 2])
    assert q.is_contiguous() and q.shape == (n, H, D)


def test_bf16_rounds_where_the_reference_rounds():
    """bf16 activations: cos and sin are rounded to bf16 and every product and sum is rounded,
    so the result differs from the fp32 computation rounded once - by a few bf16 ulps at most."""
    g = torch.Generator().manual_seed(5)
    H, D, n = 2, 64, 9
    x = torch.randn(n, 3 * H * D, generator=g)
    w, b = torch.randn(D, generator=g), 0.1 * torch.randn(D, generator=g)
    fr = _freqs(n, D, seed=6)
    q32, k32, _ = prepare_qkv(x.to(torch.bfloat16).float(), H, D, (w.bfloat16().float(), b.bfloat16().float()),
                              (w.bfloat16().float(), b.bfloat16().float()), fr)
    q16, k16, _ = prepare_qkv(x.to(torch.bfloat16), H, D, (w.bfloat16(), b.bfloat16()), (w.bfloat16(), b.bfloat16()), fr)
    assert q16.dtype == torch.bfloat16
    err = (q16.float() - q32).abs() / q32.abs().clamp_min(1.0)
    assert 0 < err.max().item() < 4 * 2 ** -8


def test_rope2d_identity_explicit_rotation_and_separation():
    g = torch.Generator().manual_seed(8)
    B, H, N, D = 1, 2, 12, 64
    x = torch.randn(B, H, N, D, generator=g, dtype=torch.float64)
    zero = torch.zeros(B, N, 2, dtype=torch.long)
    assert torch.equal(rope2d(x, zero), x)
    pos = torch.stack([torch.randint(0, N, (N,), generator=g), torch.randint(0, N, (N,), generator=g)], -1)[None]
    y = rope2d(x, pos)
    want = torch.empty_like(x)
    for n in range(N):
        for half in range(2):                      # 0: vertical (y), 1: horizontal (x)
            p = float(pos[0, n, half])
            for j in range(16):
                ang = p * 100.0 ** (-(2 * j) / 32)
                a, b = x[0, :, n, half * 32 + j], x[0, :, n, half * 32 + j + 16]
                want[0, :, n, half * 32 + j] = a * math.cos(ang) - b * math.sin(ang)
                want[0, :, n, half * 32 + j + 16] = b * math.cos(ang) + a * math.sin(ang)
    # the table's angles go through float32 (inv_freq is computed in float32)
    assert (y - want).abs().max().item() < 1e-5
    pair = lambda t: torch.stack([t[..., :16], t[..., 16:32], t[..., 32:48], t[..., 48:]], -1)
    n_in = (pair(x)[..., 0] ** 2 + pair(x)[..., 1] ** 2).sqrt()
    n_out = (pair(y)[..., 0] ** 2 + pair(y)[..., 1] ** 2).sqrt()
    assert (n_in - n_out).abs().max().item() < 1e-6
    only_y = pos.clone(); only_y[..., 1] = 0
    assert torch.equal(rope2d(x, only_y)[..., :32], y[..., :32])
    assert torch.equal(rope2d(x, only_y)[..., 32:], x[..., 32:])


def test_residual_norm_closed_forms_and_float64_restatement():
    from oracle.block_ops import residual_norm
    g = torch.Generator().manual_seed(9)
    rows, C = 5, 1024
    x, y = torch.randn(rows, C, generator=g), torch.randn(rows, C, generator=g)
    gamma, w, b = torch.randn(C, generator=g), torch.randn(C, generator=g), torch.randn(C, generator=g)
    assert torch.equal(residual_norm(x, y, torch.zeros(C))[0], x)
    assert torch.equal(residual_norm(x, y, torch.ones(C))[0], x + y)
    assert torch.equal(residual_norm(x, y, None)[0], x + y)
    xn, n = residual_norm(x, y, gamma, w, b, 1e-5)
    want = x.double() + y.double() * gamma.double()
    assert (xn.double() - want).abs().max().item() < 1e-6
    mean = want.mean(-1, keepdim=True)
    var = ((want - mean) ** 2).mean(-1, keepdim=True)
    assert (n.double() - ((want - mean) / torch.sqrt(var + 1e-5) * w.double() + b.double())).abs().max().item() < 1e-5
    # an update that makes the row constant: the LayerNorm is the bias
    _, n = residual_norm(x, 3.0 - x, torch.ones(C), w, b, 1e-5)
    assert (n - b).abs().max().item() < 2e-3     # (x + (3 - x)) is 3 up to fp32 rounding of the sum


def test_rope3d_table_hand_written_entries_and_structure():
    """518x378 frames: 27 x 37 patches after 6 special tokens; pairs 0-9 follow the frame,
    10-20 the row, 21-31 the column; each entry is exp(i * coordinate * 10000^(-2j/dim))."""
    from oracle.prepare_qkv import rope3d_freqs
    pph, ppw, s = 27, 37, 6
    n = s + pph * ppw
    t = rope3d_freqs(2, pph, ppw, s, f_start=40, f_end=42)
    assert t.shape == (1, 1, 2 * n, 32) and t.dtype == torch.complex128
    assert (t.abs() - 1).abs().max().item() < 1e-15

    def expect(coord, j, dim):
        a = coord * 10000.0 ** (-2.0 * j / dim)
        return complex(math.cos(a), math.sin(a))

    def close(z, w):
        return abs(complex(z) - w) < 1e-12

    cam0 = t[0, 0, 0]                       # camera token of frame 40: (40, 0, 0)
    assert close(cam0[0], expect(40, 0, 20)) and close(cam0[9], expect(40, 9, 20))
    assert close(cam0[10], 1.0) and close(cam0[31], 1.0)
    reg3 = t[0, 0, n + 3]                   # special token 3 of frame 41: (41, 3, 3)
    assert close(reg3[4], expect(41, 4, 20)) and close(reg3[10 + 2], expect(3, 2, 22)) and close(reg3[21 + 7], expect(3, 7, 22))
    p = t[0, 0, s + 5 * ppw + 11]           # patch (5, 11) of frame 40: (40, 6 + 5, 6 + 11)
    assert close(p[10 + 1], expect(11, 1, 22)) and close(p[21 + 10], expect(17, 10, 22)) and close(p[3], expect(40, 3, 20))
    last = t[0, 0, 2 * n - 1]               # patch (26, 36) of frame 41
    assert close(last[10], expect(32, 0, 22)) and close(last[21], expect(42, 0, 22)) and close(last[0], expect(41, 0, 20))

    # the frame index moves the frame pairs only; a one-frame table is the first frame of a longer one
    u = rope3d_freqs(2, pph, ppw, s, f_start=7, f_end=9)
    assert torch.equal(u[..., 10:], t[..., 10:]) and not torch.equal(u[..., :10], t[..., :10])
    one = rope3d_freqs(1, pph, ppw, s)
    two = rope3d_freqs(2, pph, ppw, s)
    assert torch.equal(two[:, :, :n], one) and one[0, 0, 0].eq(1).all()
    # without special tokens the grid starts at (0, 0)
    z = rope3d_freqs(1, 3, 4, 0)
    assert z.shape == (1, 1, 12, 32) and z[0, 0, 0].eq(1).all() and close(z[0, 0, 1 * 4 + 2][10 + 1], expect(1, 1, 22))
    assert close(z[0, 0, 1 * 4 + 2][21 + 1], expect(2, 1, 22))


def test_linear_epilogue_closed_forms():
    """Pins of oracle.block_ops.linear_epilogue that a dropped bias, a transposed weight, the tanh
    approximation or a missing rounding would fail."""
    from oracle.block_ops import LINEAR_BIAS, LINEAR_BIAS_GELU, LINEAR_BIAS_RESIDUAL, linear_epilogue
    g = torch.Generator().manual_seed(4)
    bf = lambda t: t.to(torch.bfloat16)
    a = bf(torch.randn(5, 8, generator=g))
    bias = bf(torch.randn(8, generator=g))
    eye = bf(torch.eye(8))
    # identity weight: the input plus the bias, rounded once
    assert torch.equal(linear_epilogue(a, eye, bias, LINEAR_BIAS), bf(a.float() + bias.float()).float())
    # a 3 x 2 weight against three float64 loops (w is [N, K]: out[m][n] = sum_k a[m][k] w[n][k])
    w = bf(torch.randn(3, 8, generator=g))
    want = torch.zeros(5, 3, dtype=torch.float64)
    for m in range(5):
        for n in range(3):
            for k in range(8):
                want[m, n] += float(a[m, k]) * float(w[n, k])
    got = linear_epilogue(a, w, None, LINEAR_BIAS)
    assert (got.double() - want).abs().max().item() <= 2.0 ** -8 * want.abs().max().item()
    # exact GELU: 0 at 0, identity far right, 0 far left, odd part x / 2 + x / 2, and not the tanh form
    x = bf(torch.tensor([[0.0, 8.0, -8.0, 1.0, -1.0, 3.0, -3.0, 0.5]]))
    y = linear_epilogue(x, eye, None, LINEAR_BIAS_GELU)[0]
    assert y[0].item() == 0.0 and y[1].item() == 8.0 and abs(y[2].item()) < 1e-6
    assert abs((y[3] - y[4]).item() - 1.0) <= 2.0 ** -7 and abs((y[5] - y[6]).item() - 3.0) <= 2.0 ** -6
    assert abs(y[3].item() - 0.8413447) <= 2.0 ** -8            # Phi(1)
    # LayerScale + residual: gamma = 0 returns the residual, gamma = 1 the rounded sum
    res = bf(torch.randn(5, 8, generator=g))
    assert torch.equal(linear_epilogue(a, eye, bias, LINEAR_BIAS_RESIDUAL, torch.zeros(8), res), res.float())
    one = linear_epilogue(a, eye, bias, LINEAR_BIAS_RESIDUAL, torch.ones(8), res)
    assert torch.equal(one, bf(res.float() + bf(a.float() + bias.float()).float()).float())
    assert torch.equal(linear_epilogue(a, eye, bias, LINEAR_BIAS_RESIDUAL, None, res), one)
