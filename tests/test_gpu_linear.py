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


@pytest.mark.parametrize("M,K,Nn", [(1004, 1024, 3072), (1004, 1024, 1024), (70, 128, 64), (4016, 1024, 1024), (129, 128, 192), (1, 128, 128)])
def test_linear_bias(M, K, Nn):
    N = _native()
    a, w, bias, _ = _inputs(M, K, Nn, seed=M + Nn)
    check(run_linear(a, w, bias, N.LINEAR_BIAS), expected(a, w, bias, N.LINEAR_BIAS))
    check(run_linear(a, w, None, N.LINEAR_BIAS), expected(a, w, None, N.LINEAR_BIAS))


@pytest.mark.parametrize("M,K,Nn", [(1004, 1024, 4096), (257, 256, 320)])
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


def test_mlp_with_fused_fc1_gelu_equals_the_unfused_module():
    """The block's Mlp takes the fused kernel for one frame's rows in bf16 and the plain torch ops
    otherwise (fp32, tanh GELU, many rows); both give the same numbers up to one bf16 ulp of the
    hidden activations."""
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
        # not taken: fp32 activations, the tanh approximation, more rows than one frame
        assert not mlp._can_fuse_fc1(x.float())
        assert not Mlp(256, 1024, act_layer=lambda: torch.nn.GELU(approximate="tanh")).to(dev).to(torch.bfloat16)._can_fuse_fc1(x)
        assert not mlp._can_fuse_fc1(torch.zeros(4, 1004, 256, device=dev, dtype=torch.bfloat16))
