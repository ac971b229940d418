"""GPU parity of the fused pre-attention producer (lbm_qkv_prepare), through the C ABI and
through the manager, against oracle/prepare_qkv.py.

Tolerances.  v, and q/k without LayerNorm: bit-exact (copies, or the reference's own sequence
of bf16 roundings).  With the per-head LayerNorm the fp32 sums inside it may be taken in a
different order than torch's, which can move a result by one bf16 ulp: at most 2^-7 relative
to max(1, |ref|) on any element and fewer than 1 element in 1000 different at all.  fp32
activations: 2e-6 relative to max(1, |ref|)."""
import ctypes as C
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _native():
    from lingbot_map_amd import _native as N
    return N


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _inputs(n, H, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    qkv = torch.randn(n, 3 * H * D, generator=g).to(dtype)
    w = [(1 + 0.2 * torch.randn(D, generator=g)).to(dtype) for _ in range(2)]
    b = [(0.1 * torch.randn(D, generator=g)).to(dtype) for _ in range(2)]
    ang = torch.rand(1, 1, n, D // 2, generator=g) * 2 * math.pi
    freqs = torch.polar(torch.ones_like(ang), ang)
    return qkv, (w[0], b[0]), (w[1], b[1]), freqs


def run_prepare(qkv, H, D, qn, kn, freqs, dst_dtype, pool=None, rows=None, page_size=16, want_kv=True, eps=1e-5,
                table=None, q_scale=1.0):
    """freqs: complex table of the interleaved embedding; table: [n, D, 2] (cos, sin) of the half-split one."""
    N = _native()
    dev = torch.device("cuda:0")
    n = qkv.shape[0]
    dt = lambda d: N.DTYPE_BF16 if d == torch.bfloat16 else N.DTYPE_F32
    f32 = lambda t: t.float().to(dev).contiguous()
    keep = [f32(t) for t in (qn or ()) + (kn or ())]
    cs = torch.view_as_real(freqs).reshape(n, D // 2, 2).float().contiguous().to(dev) if freqs is not None else None
    layout = N.ROPE_INTERLEAVED
    if table is not None:
        cs, layout = table.float().contiguous().to(dev), N.ROPE_HALF_SPLIT
    q = torch.full((n, H, D), float("nan"), dtype=dst_dtype, device=dev)
    k = torch.full_like(q, float("nan")) if want_kv else None
    v = torch.full_like(q, float("nan")) if want_kv else None
    x = qkv.to(dev)
    N.check(N.lib.lbm_qkv_prepare(ptr(x), dt(qkv.dtype), *( [ptr(t) for t in keep] if keep else [None] * 4), eps, q_scale, ptr(cs), layout,
                                  ptr(q), ptr(k), ptr(v), dt(dst_dtype), ptr(pool), ptr(rows), n, H, D, page_size, None))
    torch.cuda.synchronize()
    return q, k, v


def _close(got, ref, dtype):
    got, ref = got.float().cpu(), ref.float()
    rel = (got - ref).abs() / ref.abs().clamp_min(1.0)
    if dtype == torch.bfloat16:
        assert rel.max().item() <= 2 ** -7, rel.max().item()
        assert (got != ref).float().mean().item() < 1e-3
    else:
        assert rel.max().item() <= 2e-6, rel.max().item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,H", [(5, 2), (1004, 16)])
def test_prepare_matches_oracle(dtype, n, H):
    from oracle.prepare_qkv import prepare_qkv
    D = 64
    qkv, qn, kn, freqs = _inputs(n, H, D, dtype, seed=n + H)
    rq, rk, rv = prepare_qkv(qkv, H, D, qn, kn, freqs)
    q, k, v = run_prepare(qkv, H, D, qn, kn, freqs, dtype)
    assert torch.equal(v.cpu(), rv)
    _close(q, rq, dtype)
    _close(k, rk, dtype)


def test_prepare_without_norm_is_bit_exact_in_bf16():
    """No LayerNorm: only the reference's own sequence of bf16 roundings is left."""
    from oracle.prepare_qkv import prepare_qkv
    n, H, D = 333, 4, 64
    qkv, _, _, freqs = _inputs(n, H, D, torch.bfloat16, seed=7)
    rq, rk, rv = prepare_qkv(qkv, H, D, None, None, freqs)
    q, k, v = run_prepare(qkv, H, D, None, None, freqs, torch.bfloat16)
    assert torch.equal(q.cpu(), rq) and torch.equal(k.cpu(), rk) and torch.equal(v.cpu(), rv)
    # and with neither norm nor rope it is the layout change alone
    rq, rk, rv = prepare_qkv(qkv, H, D)
    q, k, v = run_prepare(qkv, H, D, None, None, None, torch.bfloat16)
    assert torch.equal(q.cpu(), rq) and torch.equal(k.cpu(), rk) and torch.equal(v.cpu(), rv)


def test_prepare_q_scale_rounds_the_scaled_row_once():
    """``q_scale``: q is multiplied in fp32 before its last rounding, k and v are left alone.  A power
    of two commutes with the rounding (bit-equal to the plain q times it); for sm_scale * log2(e)
    the bf16 q must be the nearest bf16 to the scaled fp32 row, which the fp32 oracle provides up
    to the rounding of the operations before the last one (one ulp)."""
    from oracle.prepare_qkv import prepare_qkv
    N = _native()
    n, H, D = 257, 4, 64
    for qn_on, rope_on in ((True, True), (False, True), (True, False), (False, False)):
        qkv, qn, kn, freqs = _inputs(n, H, D, torch.bfloat16, seed=21)
        qn, kn, freqs = (qn if qn_on else None), (kn if qn_on else None), (freqs if rope_on else None)
        q1, k1, v1 = run_prepare(qkv, H, D, qn, kn, freqs, torch.bfloat16)
        qh, kh, vh = run_prepare(qkv, H, D, qn, kn, freqs, torch.bfloat16, q_scale=0.25)
        assert torch.equal(qh.float(), q1.float() * 0.25) and torch.equal(kh, k1) and torch.equal(vh, v1)
        c = N.q_scale_log2(1.0 / math.sqrt(D))
        qc, kc, vc = run_prepare(qkv, H, D, qn, kn, freqs, torch.bfloat16, q_scale=c)
        assert torch.equal(kc, k1) and torch.equal(vc, v1)
        # against the reference's rounded q times c: half a bf16 step of either value apart at most
        ref = q1.float().cpu() * c
        got = qc.float().cpu()
        step = lambda t: torch.exp2(torch.floor(torch.log2(t.abs().clamp_min(1e-30))) - 7)
        assert ((got - ref).abs() <= 0.505 * (step(got) + c * step(q1.float().cpu()))).all()
        # and nearer to the unrounded row (fp32 oracle) than the twice-rounded c * q is, on average
        f32 = lambda t: None if t is None else tuple(x.float() for x in t)
        exact = prepare_qkv(qkv.float(), H, D, f32(qn), f32(kn), freqs)[0] * c
        twice = (q1.float().cpu() * c).to(torch.bfloat16).float()
        if qn_on or rope_on:
            assert (got - exact).abs().mean() < (twice - exact).abs().mean()
    # fp32 activations and cache: a plain multiply
    qkv, qn, kn, freqs = _inputs(33, 2, D, torch.float32, seed=22)
    q1, _, _ = run_prepare(qkv, 2, D, qn, kn, freqs, torch.float32)
    qc, _, _ = run_prepare(qkv, 2, D, qn, kn, freqs, torch.float32, q_scale=c)
    assert torch.allclose(qc, q1 * c, rtol=2e-7, atol=0)
    # refused: zero or negative
    dev = torch.device("cuda:0")
    x = torch.zeros(4, 3 * 2 * 64, dtype=torch.bfloat16, device=dev)
    q = torch.zeros(4, 2, 64, dtype=torch.bfloat16, device=dev)
    for bad in (0.0, -1.0, float("nan")):
        assert N.lib.lbm_qkv_prepare(ptr(x), 0, None, None, None, None, 1e-5, bad, None, 0, ptr(q), None, None, 0, None, None,
                                     4, 2, 64, 16, None) == N.ERR_INVALID


def test_prepare_writes_the_pool_rows_and_respects_the_gate():
    from oracle.prepare_qkv import prepare_qkv
    dev = torch.device("cuda:0")
    n, H, D, S = 40, 2, 64, 8
    qkv, qn, kn, freqs = _inputs(n, H, D, torch.bfloat16, seed=11)
    _, rk, rv = prepare_qkv(qkv, H, D, qn, kn, freqs)
    pages = 12
    pool = torch.full((pages, 2, S, H, D), 7.0, dtype=torch.bfloat16, device=dev)
    g = torch.Generator().manual_seed(3)
    slots = torch.randperm(pages * S, generator=g)[:n]
    rows = ((slots // S) * 2 * S + slots % S).to(torch.int32)
    rows[::5] = -1                                         # gated off
    q, k, v = run_prepare(qkv, H, D, qn, kn, freqs, torch.bfloat16, pool=pool, rows=rows.to(dev), page_size=S, want_kv=False)
    assert k is None and v is None
    flat = pool.cpu().view(pages, 2, S, H, D)
    written = torch.zeros(pages, S, dtype=torch.bool)
    for t in range(n):
        if rows[t] < 0:
            continue
        p, s = int(slots[t]) // S, int(slots[t]) % S
        written[p, s] = True
        _close(flat[p, 0, s], rk[t], torch.bfloat16)
        assert torch.equal(flat[p, 1, s], rv[t])
    untouched = flat[:, :, :, :, :].permute(0, 2, 1, 3, 4)[~written]
    assert (untouched == 7.0).all()


def test_prepare_argument_checks():
    N = _native()
    dev = torch.device("cuda:0")
    x = torch.zeros(4, 3 * 2 * 64, dtype=torch.bfloat16, device=dev)
    q = torch.zeros(4, 2, 64, dtype=torch.bfloat16, device=dev)
    call = lambda **kw: N.lib.lbm_qkv_prepare(ptr(x), 0, None, None, None, None, 1e-5, 1.0, None, 0, ptr(q), None, None, 0, None, None,
                                              4, 2, kw.get("D", 64), 16, None)
    assert call() == N.OK
    assert call(D=128) != N.OK and b"head_dim 64" in N.lib.lbm_last_error()
    w = torch.ones(64, device=dev)
    rc = N.lib.lbm_qkv_prepare(ptr(x), 0, ptr(w), None, None, None, 1e-5, 1.0, None, 0, ptr(q), None, None, 0, None, None, 4, 2, 64, 16, None)
    assert rc != N.OK
    torch.cuda.synchronize()


def test_manager_step_qkv_equals_step():
    """The fused producer in front of the cache gives the frames `step` gives when fed the
    oracle's q, k, v: same tables, same pool contents (k within one ulp), same attention."""
    from lingbot_map_amd import HipPagedKVCacheManager
    from oracle.prepare_qkv import prepare_qkv
    dev = torch.device("cuda:0")
    T, H, D = 70, 2, 64
    mk = lambda: HipPagedKVCacheManager(2, 8, T, H, D, torch.bfloat16, dev, num_special_tokens=5, scale_frames=1,
                                        sliding_window=3, max_total_frames=32, page_size=16, layout="frame_pages")
    a, b = mk(), mk()
    for f in range(9):
        keyframe = [f % 3 != 2]
        for blk in range(2):
            qkv, qn, kn, freqs = _inputs(T, H, D, torch.bfloat16, seed=100 * f + blk)
            rq, rk, rv = prepare_qkv(qkv, H, D, qn, kn, freqs)
            ref = a.step(blk, rq.to(dev), rk.to(dev), rv.to(dev), keyframe=keyframe)
            cs = torch.view_as_real(freqs).reshape(T, D // 2, 2).float().to(dev)
            out = b.step_qkv(blk, qkv.to(dev), (qn[0].to(dev), qn[1].to(dev)), (kn[0].to(dev), kn[1].to(dev)), cs,
                             keyframe=keyframe)
            err = (out.float() - ref.float()).abs()
            assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3
    assert a.build_visible_page_table(0) == b.build_visible_page_table(0)
    assert a.get_cache_stats(0) == b.get_cache_stats(0)
    pa, pb = a.kv_caches[1].float(), b.kv_caches[1].float()
    assert ((pa - pb).abs() / pa.abs().clamp_min(1.0)).max().item() <= 2 ** -7
    assert a.device_header()["error"] == 0 and b.device_header()["error"] == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_prepare_half_split_rope_matches_oracle(dtype):
    """The 2-D embedding of the frame blocks: pairs (j, j + 16) in each half of head_dim."""
    from lingbot_map_amd import RotaryPositionEmbedding2D
    from oracle.prepare_qkv import prepare_qkv
    n, H, D = 300, 4, 64
    qkv, qn, kn, _ = _inputs(n, H, D, dtype, seed=31)
    g = torch.Generator().manual_seed(32)
    pos = torch.stack([torch.randint(0, 27, (n,), generator=g), torch.randint(0, 37, (n,), generator=g)], -1)
    rq, rk, rv = prepare_qkv(qkv, H, D, qn, kn, None, positions=pos)
    table = RotaryPositionEmbedding2D().cos_sin_table(pos[None], D, dtype)
    q, k, v = run_prepare(qkv, H, D, qn, kn, None, dtype, table=table)
    assert torch.equal(v.cpu(), rv)
    _close(q, rq, dtype)
    _close(k, rk, dtype)
    if dtype == torch.bfloat16:     # without LayerNorm: the reference's own roundings, bit for bit
        rq, rk, _ = prepare_qkv(qkv, H, D, None, None, None, positions=pos)
        q, k, _ = run_prepare(qkv, H, D, None, None, None, dtype, table=table)
        assert torch.equal(q.cpu(), rq) and torch.equal(k.cpu(), rk)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,C", [(3, 256), (1004, 1024), (6, 1536), (5, 2048), (17, 2048 + 8), (2, 8192)])
def test_residual_norm_matches_oracle(dtype, rows, C):
    """x + y * gamma and the LayerNorm of it in one kernel.  bf16: x_out bit-exact (products and
    sums rounded where torch rounds them), the LayerNorm within one bf16 ulp; fp32: 2e-6."""
    from oracle.block_ops import residual_norm
    N = _native()
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(rows + C)
    x, y = (torch.randn(rows, C, generator=g).to(dtype) for _ in range(2))
    gamma = (0.1 * torch.randn(C, generator=g)).to(dtype)
    w, b = (1 + 0.2 * torch.randn(C, generator=g)).to(dtype), (0.1 * torch.randn(C, generator=g)).to(dtype)
    rx, rn = residual_norm(x, y, gamma, w, b, 1e-5)
    dt = N.DTYPE_BF16 if dtype == torch.bfloat16 else N.DTYPE_F32
    xd, yd = x.to(dev), y.to(dev)
    f32 = [t.float().to(dev) for t in (gamma, w, b)]
    xo, no = torch.full_like(xd, float("nan")), torch.full_like(xd, float("nan"))
    N.check(N.lib.lbm_residual_norm(ptr(xd), ptr(yd), dt, ptr(f32[0]), ptr(f32[1]), ptr(f32[2]), 1e-5, ptr(xo), ptr(no),
                                    rows, C, None))
    torch.cuda.synchronize()
    if dtype == torch.bfloat16:
        assert torch.equal(xo.cpu(), rx)
    else:
        assert ((xo.cpu() - rx).abs() / rx.abs().clamp_min(1.0)).max().item() <= 2e-6
    _close(no, rn, dtype) if dtype == torch.float32 else None
    if dtype == torch.bfloat16:
        rel = (no.float().cpu() - rn.float()).abs() / rn.float().abs().clamp_min(1.0)
        assert rel.max().item() <= 2 ** -7 and (no.cpu() != rn).float().mean().item() < 2e-3
    # without LayerScale and without LayerNorm: x + y, in place
    rx2, _ = residual_norm(x, y, None)
    N.check(N.lib.lbm_residual_norm(ptr(xd), ptr(yd), dt, None, None, None, 0.0, ptr(xd), None, rows, C, None))
    torch.cuda.synchronize()
    assert torch.equal(xd.cpu(), rx2) if dtype == torch.bfloat16 else ((xd.cpu() - rx2).abs().max().item() <= 1e-6)
    # argument checks
    assert N.lib.lbm_residual_norm(ptr(xd), ptr(yd), dt, None, ptr(f32[1]), None, 0.0, ptr(xd), None, rows, C, None) != N.OK
    assert N.lib.lbm_residual_norm(ptr(xd), ptr(yd), dt, None, None, None, 0.0, ptr(xd), None, rows, 12, None) != N.OK
