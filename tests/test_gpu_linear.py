"""lbm_linear (bf16 GEMM with fused epilogues) against fp32 arithmetic on the CPU (GPU).

The reference computes these as separate bf16 torch ops (attention.py:413,554, mlp.py:35-38,
block.py:283, layer_scale.py:21-22): linear -> round -> GELU or LayerScale -> round -> residual
add -> round.  The expected values follow that sequence with the product accumulated in fp32 on
the CPU; the kernel's own fp32 accumulation order differs, so an output may land on the
neighbouring bf16 value: every element within one bf16 ulp (relative 2^-7), fewer than 2 % of
them different at all."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _native():
    from lingbot_map_amd import _native as N
    return N


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def run_linear(a, w, bias, epilogue, gamma=None, residual=None, out=None):
    N = _native()
    dev = torch.device("cuda:0")
    f32 = lambda t: None if t is None else t.float().to(dev).contiguous()
    a_d, w_d = a.to(dev).contiguous(), w.to(dev).contiguous()
    b_d, g_d = f32(bias), f32(gamma)
    r_d = None if residual is None else residual.to(dev).contiguous()
    M, K = a.shape
    Nn = w.shape[0]
    o = torch.full((M, Nn), float("nan"), dtype=torch.bfloat16, device=dev) if out is None else out
    N.check(N.lib.lbm_linear(ptr(a_d), ptr(w_d), ptr(b_d), ptr(g_d), ptr(r_d), ptr(o), M, Nn, K, epilogue, None))
    torch.cuda.synchronize()
    return o.cpu()


def expected(a, w, bias, epilogue, gamma=None, residual=None):
    from oracle.block_ops import linear_epilogue
    return linear_epilogue(a, w, bias, epilogue, gamma, residual)


def check(got, ref, scale=None, bar=2.0 ** -7):
    """``scale``: the magnitudes the one-ulp bar refers to when they are not the outputs' own."""
    got, ref = got.float(), ref.float()
    assert torch.isfinite(got).all()
    rel = (got - ref).abs() / (ref if scale is None else scale).abs().clamp_min(2.0 ** -6)
    assert rel.max().item() <= bar, rel.max().item()
    assert (got != ref).float().mean().item() < 0.02, (got != ref).float().mean().item()


def _inputs(M, K, Nn, seed, with_bias=True):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(Nn, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    bias = (0.1 * torch.randn(Nn, generator=g)).to(torch.bfloat16) if with_bias else None
    return a, w, bias, g


# (the 4016- and 2100-row launches into 3072 / 4096 columns run on the 256 x 256 tiles)
@pytest.mark.parametrize("M,K,Nn", [(1004, 1024, 3072), (1004, 1024, 1024), (70, 128, 64), (4016, 1024, 1024), (129, 128, 192), (1, 128, 128),
                                    (4016, 1024, 3072), (2100, 1024, 4096), (4016, 128, 4096)])
def test_linear_bias(M, K, Nn):
    N = _native()
    a, w, bias, _ = _inputs(M, K, Nn, seed=M + Nn)
    check(run_linear(a, w, bias, N.LINEAR_BIAS), expected(a, w, bias, N.LINEAR_BIAS))
    check(run_linear(a, w, None, N.LINEAR_BIAS), expected(a, w, None, N.LINEAR_BIAS))


def test_linear_tile_counts_that_do_not_fill_rounds_of_the_cus():
    """Workgroups take tiles in blocks of 4 x 8 per XCD and in rounds of 256; shapes whose tile
    counts are not multiples of 8, 32 or 256 - one tile, a last panel narrower than 8 column tiles,
    a last round that does not give every XCD the same number of tiles, more than one round - must
    still have every tile computed exactly once.  K from the shortest loop (two 64-wide steps) up;
    both tile widths and both kernels (the last three shapes run on the 256- and 192-row tiles)."""
    N = _native()
    for M, K, Nn in [(1, 128, 64), (130, 128, 576), (700, 128, 1152), (1100, 256, 1344), (2300, 128, 2240), (5000, 128, 832),
                     (390, 384, 4288), (4500, 128, 5120), (9000, 128, 4352), (6100, 256, 3328)]:
        a, w, bias, _ = _inputs(M, K, Nn, seed=M + Nn)
        got = run_linear(a, w, bias, N.LINEAR_BIAS)
        check(got, expected(a, w, bias, N.LINEAR_BIAS))


def test_gelu_epilogue_on_every_bf16_pre_activation():
    """One-hot activations make the pre-activation of output (i, n) the weight w[n, i] itself, so
    a 512 x 128 weight matrix puts every finite bf16 bit pattern through the epilogue: the
    tabulated range, the values below and above it, both zeros, the negative tail.  torch's GELU
    of the same bf16 values is the expectation: bit-equal from -3 up (zeros compare equal whatever
    their sign), within one bf16 ulp of the pre-activation's scale below -3, where torch's result
    is the last bits of its erff (1 + erf cancels) and the table holds the exact value."""
    N = _native()
    bits = torch.arange(65536, dtype=torch.int32)
    exp_field = (bits >> 7) & 0xFF
    bits = torch.where(exp_field == 0xFF, torch.zeros_like(bits), bits)      # inf / NaN would poison the other columns' sums
    w = bits.to(torch.uint16).view(torch.bfloat16).reshape(512, 128)
    a = torch.eye(128, dtype=torch.bfloat16)
    got = run_linear(a, w, None, N.LINEAR_BIAS_GELU)                          # [128, 512]: got[i, n] = gelu(w[n, i])
    pre = w.t().contiguous()
    ref = torch.nn.functional.gelu(pre.to("cuda:0")).cpu()
    head = pre.float() >= -3.0
    assert torch.equal(got.float()[head], ref.float()[head])
    tail = ~head
    assert ((got.float() - ref.float()).abs()[tail] <= 2.0 ** -8 * 2.0 ** -7 * pre.float().abs()[tail] + 1e-30).all()


@pytest.mark.parametrize("M,K,Nn", [(1004, 1024, 4096), (257, 256, 320), (4016, 1024, 4096)])
def test_linear_bias_gelu(M, K, Nn):
    N = _native()
    a, w, bias, _ = _inputs(M, K, Nn, seed=7)
    # a pre-activation on the neighbouring bf16 value moves the output by up to 1.13 (the largest
    # slope of GELU) ulps of the PRE-activation, which for outputs near zero is many of their own
    pre = expected(a, w, bias, N.LINEAR_BIAS)
    check(run_linear(a, w, bias, N.LINEAR_BIAS_GELU), expected(a, w, bias, N.LINEAR_BIAS_GELU), scale=pre, bar=1.2 * 2.0 ** -7 + 2.0 ** -8)


@pytest.mark.parametrize("M,K,Nn,with_gamma", [(1004, 4096, 1024, True), (1004, 1024, 1024, False), (300, 256, 128, True)])
def test_linear_layerscale_residual(M, K, Nn, with_gamma):
    N = _native()
    a, w, bias, g = _inputs(M, K, Nn, seed=11)
    res = torch.randn(M, Nn, generator=g).to(torch.bfloat16)
    gamma = (0.5 + torch.rand(Nn, generator=g)).to(torch.bfloat16) if with_gamma else None
    ref = expected(a, w, bias, N.LINEAR_BIAS_RESIDUAL, gamma, res)
    # one ulp of the larger of the two addends (the sum itself may be near zero), plus the sum's own
    scale = torch.maximum(res.float().abs(), (ref - res.float()).abs())
    check(run_linear(a, w, bias, N.LINEAR_BIAS_RESIDUAL, gamma, res), ref, scale=scale, bar=2.0 ** -6)
    # in place: the residual is also the output
    x = res.to("cuda:0").clone()
    a_d, w_d, b_d = a.to("cuda:0"), w.to("cuda:0"), bias.float().to("cuda:0")
    g_d = gamma.float().to("cuda:0") if with_gamma else None
    N.check(N.lib.lbm_linear(ptr(a_d), ptr(w_d), ptr(b_d), ptr(g_d), ptr(x), ptr(x), M, Nn, K, N.LINEAR_BIAS_RESIDUAL, None))
    torch.cuda.synchronize()
    check(x.cpu(), ref, scale=scale, bar=2.0 ** -6)


def test_linear_rows_past_m_are_not_written_and_arguments_are_checked():
    N = _native()
    a, w, bias, _ = _inputs(200, 128, 128, seed=3)
    out = torch.full((256, 128), 7.0, dtype=torch.bfloat16, device="cuda:0")   # 56 rows of slack behind the result
    got = run_linear(a, w, bias, N.LINEAR_BIAS, out=out)
    check(got[:200], expected(a, w, bias, N.LINEAR_BIAS))
    assert torch.equal(got[200:], torch.full((56, 128), 7.0, dtype=torch.bfloat16))
    dev = "cuda:0"
    bad = lambda *args: N.lib.lbm_linear(*args) != N.OK
    o = torch.empty(200, 128, dtype=torch.bfloat16, device=dev)
    ad, wd = a.to(dev), w.to(dev)
    assert bad(ptr(ad), ptr(wd), None, None, None, ptr(o), 200, 100, 128, N.LINEAR_BIAS, None)      # N not a multiple of 64
    assert bad(ptr(ad), ptr(wd), None, None, None, ptr(o), 200, 128, 64, N.LINEAR_BIAS, None)       # K not a multiple of 128
    assert bad(ptr(ad), ptr(wd), None, None, None, ptr(o), 200, 128, 128, N.LINEAR_BIAS_RESIDUAL, None)  # no residual
    assert bad(ptr(ad), ptr(wd), None, None, ptr(o), ptr(o), 200, 128, 128, N.LINEAR_BIAS, None)    # residual without the epilogue
    assert bad(ptr(ad), ptr(wd), None, None, None, ptr(o), 200, 128, 128, 9, None)
    # no rows: accepted, nothing written
    o.fill_(3.0)
    N.check(N.lib.lbm_linear(ptr(ad), ptr(wd), None, None, None, ptr(o), 0, 128, 128, N.LINEAR_BIAS, None))
    N.check(N.lib.lbm_qkv_linear_prepare(ptr(ad), ptr(wd), None, 0, 128, None, None, None, None, 1e-5, 1.0, None, 0, ptr(o), None, None,
                                         None, None, 2, 64, 16, None))
    torch.cuda.synchronize()
    assert bool((o == 3.0).all())


def test_mlp_with_fused_fc1_gelu_equals_the_unfused_module():
    """The block's Mlp takes the fused kernel for bf16 rows (one frame's or several streams') and the
    plain torch ops otherwise (fp32, tanh GELU); both give the same numbers up to one bf16 ulp of
    the hidden activations."""
    from lingbot_map_amd.block import Mlp
    torch.manual_seed(0)
    dev = torch.device("cuda:0")
    mlp = Mlp(256, 1024).to(dev).to(torch.bfloat16).eval()
    x = torch.randn(2, 150, 256, device=dev).to(torch.bfloat16)
    with torch.no_grad():
        assert mlp._can_fuse_fc1(x)
        hidden = mlp.fc1_gelu(x)
        ref_hidden = mlp.act(mlp.fc1(x))
        pre = mlp.fc1(x)
        check(hidden.cpu(), ref_hidden.cpu(), scale=pre.cpu(), bar=1.2 * 2.0 ** -7 + 2.0 ** -8)
        out, ref = mlp(x), mlp.fc2(ref_hidden)
        assert (out.float() - ref.float()).abs().max().item() <= 2.0 ** -6 * ref.float().abs().max().item()
        # not taken: fp32 activations, the tanh approximation; taken: four streams' rows
        assert not mlp._can_fuse_fc1(x.float())
        assert not Mlp(256, 1024, act_layer=lambda: torch.nn.GELU(approximate="tanh")).to(dev).to(torch.bfloat16)._can_fuse_fc1(x)
        many = torch.randn(4, 1004, 256, device=dev).to(torch.bfloat16)
        assert mlp._can_fuse_fc1(many)
        check(mlp.fc1_gelu(many).cpu(), mlp.act(mlp.fc1(many)).cpu(), scale=mlp.fc1(many).cpu(), bar=1.2 * 2.0 ** -7 + 2.0 ** -8)


@pytest.mark.parametrize("rope", ["none", "interleaved", "half_split"])
@pytest.mark.parametrize("norm", [False, True])
@pytest.mark.parametrize("M,H,K", [(1004, 16, 1024), (70, 3, 128), (4016, 16, 1024), (3900, 16, 256)])
def test_qkv_projection_with_the_producer_as_its_epilogue(M, H, K, norm, rope):
    """lbm_qkv_linear_prepare against lbm_linear (bias) followed by lbm_qkv_prepare on its output:
    the same arithmetic on the same rounded projection, so q, k, v and the pool rows are bit-equal.
    Keyframe-gated pool writes (some rows -1), k_out / v_out present and absent, an odd number of
    heads (64-column tiles)."""
    N = _native()
    dev = torch.device("cuda:0")
    D, S = 64, 16
    g = torch.Generator().manual_seed(M + H + K + norm + len(rope))
    a = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(3 * H * D, K, generator=g) / K ** 0.5).to(torch.bfloat16).to(dev)
    bias = (0.1 * torch.randn(3 * H * D, generator=g)).to(dev)
    ln = [(1 + 0.2 * torch.randn(D, generator=g)).to(dev) if i % 2 == 0 else (0.1 * torch.randn(D, generator=g)).to(dev)
          for i in range(4)] if norm else [None] * 4
    cs, layout = None, N.ROPE_INTERLEAVED
    if rope == "interleaved":
        ang = torch.rand(M, D // 2, generator=g) * 6.283185
        cs = torch.stack([ang.cos(), ang.sin()], dim=-1).contiguous().to(dev)
    elif rope == "half_split":
        ang = torch.rand(M, D, generator=g) * 6.283185
        cs, layout = torch.stack([ang.cos(), ang.sin()], dim=-1).contiguous().to(dev), N.ROPE_HALF_SPLIT
    n_pages = -(-M // S) + 3
    rows = torch.randperm(n_pages * S, generator=g)[:M]
    rows = ((rows // S) * 2 * S + rows % S).to(torch.int32)
    rows[::7] = -1                                            # gated off
    rows = rows.to(dev)
    for with_kv, with_pool in ((True, True), (False, True), (True, False)):
        def outputs():
            q = torch.full((M, H, D), float("nan"), dtype=torch.bfloat16, device=dev)
            k = torch.full_like(q, float("nan")) if with_kv else None
            v = torch.full_like(q, float("nan")) if with_kv else None
            pool = torch.zeros(n_pages, 2, S, H, D, dtype=torch.bfloat16, device=dev) if with_pool else None
            return q, k, v, pool
        q0, k0, v0, pool0 = outputs()
        qkv = torch.empty(M, 3 * H * D, dtype=torch.bfloat16, device=dev)
        N.check(N.lib.lbm_linear(ptr(a), ptr(w), ptr(bias), None, None, ptr(qkv), M, 3 * H * D, K, N.LINEAR_BIAS, None))
        N.check(N.lib.lbm_qkv_prepare(ptr(qkv), N.DTYPE_BF16, *[ptr(t) for t in ln], 1e-5, 1.0, ptr(cs), layout, ptr(q0), ptr(k0), ptr(v0),
                                      N.DTYPE_BF16, ptr(pool0), ptr(rows) if with_pool else None, M, H, D, S, None))
        q1, k1, v1, pool1 = outputs()
        N.check(N.lib.lbm_qkv_linear_prepare(ptr(a), ptr(w), ptr(bias), M, K, *[ptr(t) for t in ln], 1e-5, 1.0, ptr(cs), layout,
                                             ptr(q1), ptr(k1), ptr(v1), ptr(pool1), ptr(rows) if with_pool else None, H, D, S, None))
        torch.cuda.synchronize()
        assert torch.isfinite(q1.float()).all() and torch.equal(q0, q1)
        if with_kv:
            assert torch.equal(k0, k1) and torch.equal(v0, v1)
        if with_pool:
            assert torch.equal(pool0, pool1) and pool1.float().abs().sum().item() > 0
    # argument checks
    bad = lambda *args: N.lib.lbm_qkv_linear_prepare(*args) != N.OK
    q1 = torch.empty(M, H, D, dtype=torch.bfloat16, device=dev)
    assert bad(ptr(a), ptr(w), None, M, K, None, None, None, None, 1e-5, 1.0, None, 0, ptr(q1), None, None, None, None, H, 128, S, None)   # head_dim
    assert bad(ptr(a), ptr(w), None, M, K, ptr(bias), None, None, None, 1e-5, 1.0, None, 0, ptr(q1), None, None, None, None, H, D, S, None)  # one norm parameter
    assert bad(ptr(a), ptr(w), None, M, K, None, None, None, None, 1e-5, 1.0, None, 0, ptr(q1), None, None, None, ptr(rows), H, D, S, None)  # rows without pool


def _row_norm(N, stats, colsum, tiles, eps=1e-5):
    return N.RowNorm(stats.data_ptr(), colsum.data_ptr(), tiles, eps)


def _fold(lw, lb, w, bias):
    """The LayerNorm's weight and bias folded into a linear layer, as lbm_row_norm asks the caller
    to: weight (bf16), its row sums (of the rounded values), bias."""
    wf = (w.float() * lw.float()[None, :]).to(torch.bfloat16)
    return wf, wf.float().sum(dim=1).contiguous(), (bias.float() + w.float() @ lb.float()).contiguous()


@pytest.mark.parametrize("M,K,Nn", [(1004, 4096, 1024), (1004, 1024, 1024), (130, 256, 256), (1, 128, 64)])
def test_residual_epilogue_leaves_row_statistics(M, K, Nn):
    """out_stats of the residual epilogue: per row and column tile the mean and the sum of squared
    deviations of the bf16 values the launch stored, against float64 on those values; the output
    itself is the one lbm_linear gives."""
    N = _native()
    dev = torch.device("cuda:0")
    a, w, bias, g = _inputs(M, K, Nn, seed=3 * M + Nn)
    gamma = torch.randn(Nn, generator=g)
    res = torch.randn(M, Nn, generator=g).to(torch.bfloat16)
    plain = run_linear(a, w, bias, N.LINEAR_BIAS_RESIDUAL, gamma=gamma, residual=res)
    tiles = N.lib.lbm_linear_stats_tiles(M, Nn)
    assert tiles in (Nn // 64, Nn // 128)
    out = torch.full((M, Nn), float("nan"), dtype=torch.bfloat16, device=dev)
    stats = torch.full((M, tiles, 2), float("nan"), dtype=torch.float32, device=dev)
    ad, wd, bd, gd, rd = a.to(dev), w.to(dev), bias.float().to(dev), gamma.float().to(dev), res.to(dev)
    N.check(N.lib.lbm_linear_norm(ptr(ad), None, ptr(wd), ptr(bd), ptr(gd), ptr(rd), ptr(out), ptr(stats), M, Nn, K,
                                  N.LINEAR_BIAS_RESIDUAL, None, 0, None))
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), plain)
    x = out.cpu().double().reshape(M, tiles, Nn // tiles)
    mean = x.mean(dim=-1)
    m2 = ((x - mean[..., None]) ** 2).sum(dim=-1)
    got = stats.cpu().double()
    assert (got[..., 0] - mean).abs().max().item() <= 1e-5 * max(1.0, mean.abs().max().item())
    assert ((got[..., 1] - m2).abs() <= 1e-4 * m2.clamp_min(1e-3)).all()
    # statistics only come with the residual epilogue, a folded LayerNorm never with it
    assert N.lib.lbm_linear_norm(ptr(ad), None, ptr(wd), ptr(bd), None, None, ptr(out), ptr(stats), M, Nn, K, N.LINEAR_BIAS, None, 0, None) != N.OK
    ln = _row_norm(N, stats, gd, tiles)
    assert N.lib.lbm_linear_norm(ptr(ad), ln, ptr(wd), ptr(bd), ptr(gd), ptr(rd), ptr(out), None, M, Nn, K, N.LINEAR_BIAS_RESIDUAL, None, 0, None) != N.OK


def _stats_of(x, tiles):
    """(mean, M2) per row and column tile of a bf16 matrix, as the residual epilogue leaves them."""
    xs = x.float().reshape(x.shape[0], tiles, -1)
    mean = xs.mean(dim=-1)
    return torch.stack([mean, ((xs - mean[..., None]) ** 2).sum(dim=-1)], dim=-1).contiguous()


@pytest.mark.parametrize("M,K,Nn,tiles,epilogue", [(1004, 1024, 4096, 16, 1), (1004, 1024, 3072, 8, 0), (200, 256, 128, 4, 1),
                                                   (77, 2048, 64, 32, 0), (4016, 1024, 4096, 8, 1), (4016, 1024, 3072, 16, 0),
                                                   (2050, 2048, 4096, 32, 0)])
def test_layernorm_folded_into_the_linear(M, K, Nn, tiles, epilogue):
    """lbm_linear_norm with a_norm (the LayerNorm's affine part folded into weight and bias by the
    caller) against LayerNorm (torch, bf16 in and out) followed by the plain lbm_linear arithmetic
    on the CPU.  The two round in different places - the normalised rows there, the folded weights
    here - so the two differ by the accumulated rounding noise of 1,024 products (a few 1e-3, the worst
    of millions of outputs 3e-2) on top of the output's own rounding; the mean difference stays a
    fraction of a bf16 step, and against float64 arithmetic the folded form is the closer of the two."""
    N = _native()
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(M + K + Nn)
    x = (torch.randn(M, K, generator=g) * (1 + torch.rand(M, 1, generator=g)) + 0.3 * torch.randn(M, 1, generator=g)).to(torch.bfloat16)
    lw = (1 + 0.2 * torch.randn(K, generator=g)).to(torch.bfloat16)
    lb = (0.1 * torch.randn(K, generator=g)).to(torch.bfloat16)
    w = (torch.randn(Nn, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    bias = (0.1 * torch.randn(Nn, generator=g)).to(torch.bfloat16)
    normed = torch.nn.functional.layer_norm(x.float(), (K,), lw.float(), lb.float(), 1e-5).to(torch.bfloat16)
    ref = expected(normed, w, bias, epilogue).float()
    pre = expected(normed, w, bias, N.LINEAR_BIAS).float()
    exact = torch.nn.functional.layer_norm(x.double(), (K,), lw.double(), lb.double(), 1e-5) @ w.double().t() + bias.double()
    if epilogue == N.LINEAR_BIAS_GELU:
        exact = torch.nn.functional.gelu(exact)
    wf, colsum, bf = _fold(lw, lb, w, bias)
    stats = _stats_of(x, tiles).to(dev)
    xd, wd, cd, bd = x.to(dev), wf.to(dev), colsum.to(dev), bf.to(dev)
    ln = _row_norm(N, stats, cd, tiles)
    out = torch.full((M, Nn), float("nan"), dtype=torch.bfloat16, device=dev)
    N.check(N.lib.lbm_linear_norm(ptr(xd), ln, ptr(wd), ptr(bd), None, None, ptr(out), None, M, Nn, K, epilogue, None, 0, None))
    torch.cuda.synchronize()
    got = out.cpu().float()
    assert torch.isfinite(got).all()
    err = (got - ref).abs()
    assert (err <= 2.0 ** -6 * pre.abs() + 2.0 ** -5).all(), err.max().item()       # the worst of a few million
    assert err.mean().item() <= 2.0 ** -8 * pre.abs().mean().item(), (err.mean().item(), pre.abs().mean().item())
    assert (got.double() - exact).abs().mean().item() <= 1.05 * (ref.double() - exact).abs().mean().item()
    # a tile count that does not divide K, missing column sums
    assert N.lib.lbm_linear_norm(ptr(xd), _row_norm(N, stats, cd, 7), ptr(wd), ptr(bd), None, None, ptr(out), None, M, Nn, K, epilogue, None, 0, None) != N.OK
    assert N.lib.lbm_linear_norm(ptr(xd), N.RowNorm(stats.data_ptr(), None, tiles, 1e-5), ptr(wd), ptr(bd), None, None, ptr(out), None, M, Nn, K, epilogue, None, 0, None) != N.OK


@pytest.mark.parametrize("M", [1004, 4016])
def test_layernorm_folded_into_the_qkv_projection_and_producer(M):
    """lbm_qkv_linear_prepare_norm (norm1 folded into the projection) against the same launch fed
    with the LayerNorm computed by torch: q, k, v agree to a bf16 step of the largest values, the
    mean difference a small fraction of that."""
    N = _native()
    dev = torch.device("cuda:0")
    H, K, D, S, tiles = 16, 1024, 64, 16, 16
    g = torch.Generator().manual_seed(91)
    x = (torch.randn(M, K, generator=g) * 1.7 + 0.2).to(torch.bfloat16)
    lw = (1 + 0.2 * torch.randn(K, generator=g)).to(torch.bfloat16)
    lb = (0.1 * torch.randn(K, generator=g)).to(torch.bfloat16)
    w = (torch.randn(3 * H * D, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    bias = 0.1 * torch.randn(3 * H * D, generator=g)
    qk = [(1 + 0.2 * torch.randn(D, generator=g)).to(dev) if i % 2 == 0 else (0.1 * torch.randn(D, generator=g)).to(dev) for i in range(4)]
    ang = torch.rand(M, D // 2, generator=g) * 6.283185
    cs = torch.stack([ang.cos(), ang.sin()], dim=-1).contiguous().to(dev)
    normed = torch.nn.functional.layer_norm(x.float(), (K,), lw.float(), lb.float(), 1e-5).to(torch.bfloat16).to(dev)
    wf, colsum, bf = _fold(lw, lb, w, bias)
    outs = []
    for fold in (False, True):
        q, k, v = (torch.full((M, H, D), float("nan"), dtype=torch.bfloat16, device=dev) for _ in range(3))
        if fold:
            xd, wd, cd, bd, stats = x.to(dev), wf.to(dev), colsum.to(dev), bf.to(dev), _stats_of(x, tiles).to(dev)
            ln = _row_norm(N, stats, cd, tiles)
            N.check(N.lib.lbm_qkv_linear_prepare_norm(ptr(xd), ln, ptr(wd), ptr(bd), M, K, *[ptr(t) for t in qk], 1e-5, 1.0, ptr(cs),
                                                      N.ROPE_INTERLEAVED, ptr(q), ptr(k), ptr(v), None, None, H, D, S, None))
        else:
            wd, bd = w.to(dev), bias.to(dev)
            N.check(N.lib.lbm_qkv_linear_prepare(ptr(normed), ptr(wd), ptr(bd), M, K, *[ptr(t) for t in qk], 1e-5, 1.0, ptr(cs),
                                                 N.ROPE_INTERLEAVED, ptr(q), ptr(k), ptr(v), None, None, H, D, S, None))
        torch.cuda.synchronize()
        outs.append([t.float().cpu() for t in (q, k, v)])
    for a0, a1 in zip(*outs):
        assert torch.isfinite(a1).all()
        # q and k come out of a LayerNorm over the head and a rotation that mixes pairs: the bar has
        # an absolute part for the worst of three million elements (the noise of 1,024 products, 5 sigma)
        assert ((a0 - a1).abs() <= 2.0 ** -6 * a0.abs() + 2.0 ** -4).all(), (a0 - a1).abs().max().item()
        assert (a0 - a1).abs().mean().item() <= 2.0 ** -9 * a0.abs().mean().item() + 1e-3


@pytest.mark.parametrize("M,K,Nn", [(1004, 4096, 1024), (200, 4096, 256), (130, 2048, 64)])
def test_residual_epilogue_with_k_split_over_workgroups(M, K, Nn):
    """With a workspace, launches with few tiles and a long K put several workgroups on a tile; the
    one that finishes last sums the slices in a fixed order.  Against the CPU arithmetic (same bars
    as the one-workgroup kernel), three launches in a row on one workspace (the counters go back to
    zero by themselves) giving the same bits, statistics included."""
    N = _native()
    dev = torch.device("cuda:0")
    a, w, bias, g = _inputs(M, K, Nn, seed=11 * M + Nn)
    gamma = torch.randn(Nn, generator=g)
    res = torch.randn(M, Nn, generator=g).to(torch.bfloat16)
    ref = expected(a, w, bias, N.LINEAR_BIAS_RESIDUAL, gamma=gamma, residual=res)
    need = N.lib.lbm_linear_workspace_bytes(M, Nn, K, N.LINEAR_BIAS_RESIDUAL)
    assert need > 0 and N.lib.lbm_linear_workspace_bytes(M, Nn, K, N.LINEAR_BIAS) == 0
    assert N.lib.lbm_linear_workspace_bytes(1004, 1024, 1024, N.LINEAR_BIAS_RESIDUAL) == 0      # proj: K too short to split
    ws = torch.zeros(need, dtype=torch.uint8, device=dev)
    tiles = N.lib.lbm_linear_stats_tiles(M, Nn)
    ad, wd, bd, gd, rd = a.to(dev), w.to(dev), bias.float().to(dev), gamma.float().to(dev), res.to(dev)
    outs = []
    for _ in range(3):
        out = torch.full((M, Nn), float("nan"), dtype=torch.bfloat16, device=dev)
        stats = torch.full((M, tiles, 2), float("nan"), dtype=torch.float32, device=dev)
        N.check(N.lib.lbm_linear_norm(ptr(ad), None, ptr(wd), ptr(bd), ptr(gd), ptr(rd), ptr(out), ptr(stats), M, Nn, K,
                                      N.LINEAR_BIAS_RESIDUAL, ptr(ws), need, None))
        torch.cuda.synchronize()
        outs.append((out.cpu(), stats.cpu()))
    n_tiles = ((M + 127) // 128) * tiles
    assert ws[:4 * n_tiles].view(torch.int32).abs().sum().item() == 0            # counters back at zero
    scale = torch.maximum(res.float().abs(), (ref.float() - res.float()).abs())
    check(outs[0][0], ref, scale=scale, bar=2.0 ** -6)
    for o, st in outs[1:]:
        assert torch.equal(o, outs[0][0]) and torch.equal(st, outs[0][1])
    x = outs[0][0].double().reshape(M, tiles, Nn // tiles)
    assert (outs[0][1][..., 0].double() - x.mean(-1)).abs().max().item() <= 1e-5 * max(1.0, x.mean(-1).abs().max().item())
    # a workspace that is too small: the launch runs unsplit; the residual aliasing the output is refused with a workspace
    out = torch.full((M, Nn), float("nan"), dtype=torch.bfloat16, device=dev)
    N.check(N.lib.lbm_linear_norm(ptr(ad), None, ptr(wd), ptr(bd), ptr(gd), ptr(rd), ptr(out), None, M, Nn, K,
                                  N.LINEAR_BIAS_RESIDUAL, ptr(ws), 1024, None))
    torch.cuda.synchronize()
    check(out.cpu(), ref, scale=scale, bar=2.0 ** -6)
    assert N.lib.lbm_linear_norm(ptr(ad), None, ptr(wd), ptr(bd), ptr(gd), ptr(rd), ptr(rd), None, M, Nn, K,
                                 N.LINEAR_BIAS_RESIDUAL, ptr(ws), need, None) != N.OK


@pytest.mark.parametrize("M,K,Nn,epilogue", [(1004, 1024, 3072, "bias"), (1004, 4096, 1024, "residual"), (70, 128, 64, "gelu"),
                                             (4016, 1024, 4096, "gelu"), (1004, 1024, 1024, "residual")])
def test_prefetch_hint_changes_no_result(M, K, Nn, epilogue):
    """lbm_linear_prefetch_hint: the launch that consumes a hint reads the named memory besides its
    own work - whole buffers, buffers that end inside a 128-byte line, a single line, one shorter
    than a line (ignored) - and writes what it writes without the hint, bit for bit; the 256-row
    tiles (4,016 rows into 4,096 columns) ignore the hint; a withdrawn hint is no hint."""
    N = _native()
    dev = torch.device("cuda:0")
    a, w, bias, g = _inputs(M, K, Nn, seed=M + K + Nn)
    epi = {"bias": N.LINEAR_BIAS, "gelu": N.LINEAR_BIAS_GELU, "residual": N.LINEAR_BIAS_RESIDUAL}[epilogue]
    gamma = torch.rand(Nn, generator=g).to(torch.bfloat16) if epilogue == "residual" else None
    res = torch.randn(M, Nn, generator=g).to(torch.bfloat16) if epilogue == "residual" else None
    plain = run_linear(a, w, bias, epi, gamma, res)
    big = torch.randn(3_000_000, generator=g).to(torch.bfloat16).to(dev)      # 6 MB, like a layer's weights
    for nbytes in (big.numel() * 2, 1_000_003, 128, 127):
        assert N.lib.lbm_linear_prefetch_hint(ptr(big), nbytes) == N.OK
        hinted = run_linear(a, w, bias, epi, gamma, res)
        assert torch.equal(hinted, plain), nbytes
    assert N.lib.lbm_linear_prefetch_hint(ptr(big), big.numel() * 2) == N.OK
    assert N.lib.lbm_linear_prefetch_hint(None, 0) == N.OK                     # withdrawn
    assert torch.equal(run_linear(a, w, bias, epi, gamma, res), plain)
    # through the split-K launch too (fc2 of one frame)
    need = N.lib.lbm_linear_workspace_bytes(M, Nn, K, epi)
    if need:
        f32 = lambda t: t.float().to(dev).contiguous()
        a_d, w_d, b_d, g_d, r_d = a.to(dev), w.to(dev), f32(bias), f32(gamma), res.to(dev)
        ws = torch.zeros(need, dtype=torch.uint8, device=dev)
        outs = []
        for hint in (False, True):
            o = torch.full((M, Nn), float("nan"), dtype=torch.bfloat16, device=dev)
            if hint:
                assert N.lib.lbm_linear_prefetch_hint(ptr(big), big.numel() * 2) == N.OK
            N.check(N.lib.lbm_linear_norm(ptr(a_d), None, ptr(w_d), ptr(b_d), ptr(g_d), ptr(r_d), ptr(o), None, M, Nn, K, epi,
                                          ptr(ws), need, None))
            torch.cuda.synchronize()
            outs.append(o.cpu())
        assert torch.equal(outs[0], outs[1]) and torch.isfinite(outs[0].float()).all()
