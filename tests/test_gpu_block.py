"""The streaming branch of the block on the GPU: outputs against the same block evaluated
with a dense dict cache (the reference SDPA path's semantics) and torch SDPA in fp32."""
import pytest
import torch

pytestmark = pytest.mark.gpu


class ReferenceSurfaceOnly:
    """Hides everything but the reference manager's call surface
    (lingbot_map/layers/flashinfer_cache.py:202-560)."""

    def __init__(self, m):
        object.__setattr__(self, "_m", m)

    def __getattr__(self, name):
        if name in ("step", "step_qkv", "set_active_streams"):
            raise AttributeError(name)
        return getattr(self._m, name)

    def __setattr__(self, name, value):
        setattr(self._m, name, value)


@pytest.mark.parametrize("reference_calls,rope", [(False, False), (True, False), (False, True), (True, True)])
def test_block_stream_matches_dense_cache(reference_calls, rope):
    """reference_calls=False takes the fused producer + `step_qkv`; True the reference's own
    method sequence.  rope=True adds the global blocks' 3-D rotary embedding (interleaved pairs,
    complex table per frame)."""
    from lingbot_map_amd import (HipPagedBlock, HipPagedKVCacheManager, RotaryPositionEmbedding3D, keyframe_flags,
                                 set_skip_append)
    from oracle.sdpa_cache import DictCacheOracle
    torch.manual_seed(5)
    rope3d = RotaryPositionEmbedding3D(attention_head_dim=64)
    dev = torch.device("cuda:0")
    dim, H, T, n_sp, scale, window, blocks = 256, 4, 53, 5, 1, 3, 2
    mods = [HipPagedBlock(dim, H, init_values=0.1, qk_norm=True, rope=True if rope else None,
                          kv_cache_sliding_window=window,
                          kv_cache_scale_frames=scale).to(dev, torch.bfloat16).eval() for _ in range(blocks)]
    for mod in mods:   # non-trivial LayerNorm parameters
        for ln in (mod.attn.q_norm, mod.attn.k_norm):
            ln.weight.data.uniform_(0.5, 1.5)
            ln.bias.data.uniform_(-0.2, 0.2)
    m = HipPagedKVCacheManager(blocks, scale + window + 16, T, H, 64, torch.bfloat16, dev, num_special_tokens=n_sp,
                               scale_frames=scale, sliding_window=window, max_total_frames=64, page_size=16,
                               layout="frame_pages")
    cache = ReferenceSurfaceOnly(m) if reference_calls else m
    dense = [DictCacheOracle(scale, window, n_sp) for _ in range(blocks)]
    flags = keyframe_flags(14, scale, 3)
    with torch.no_grad():
        for f, kf in enumerate(flags):
            x = torch.randn(1, T, dim, device=dev).to(torch.bfloat16)
            pos = None
            if rope:   # complex128 table of frame f: 5 special tokens + a 6 x 8 patch grid
                pos = rope3d(ppf=1, pph=6, ppw=8, patch_start_idx=n_sp, device=dev, f_start=f, f_end=f + 1)
                assert pos.shape == (1, 1, T, 32) and pos.dtype == torch.complex128
            set_skip_append(cache, not kf)
            y, y_ref = x, x
            for b, mod in enumerate(mods):
                y = mod(y, pos=pos, enable_3d_rope=rope, kv_cache=cache, global_idx=b, num_frames=1)
                q, k, v = mod.attn_pre(y_ref, pos=pos, enable_3d_rope=rope)
                kk, vv = dense[b].visible(k, v, keyframe=kf)
                a = torch.nn.functional.scaled_dot_product_attention(
                    q.float().permute(1, 0, 2)[None], kk.float().permute(1, 0, 2)[None], vv.float().permute(1, 0, 2)[None])
                a = a[0].permute(1, 0, 2).reshape(1, T, dim).to(torch.bfloat16)
                y_ref = mod.ffn_residual(y_ref + mod.ls1(mod.attn.proj(a)))
            set_skip_append(cache, False)
            err = (y.float() - y_ref.float()).abs()
            assert err.max().item() <= 3e-2 and err.mean().item() <= 2e-3, (f, err.max().item(), err.mean().item())
    assert m.frame_count == [sum(flags)] * blocks and m.device_header()["error"] == 0


def test_two_streams_through_one_block():
    from lingbot_map_amd import HipPagedBlock, HipPagedKVCacheManager
    torch.manual_seed(6)
    dev = torch.device("cuda:0")
    dim, H, T = 256, 4, 53
    mod = HipPagedBlock(dim, H, qk_norm=True, kv_cache_sliding_window=2, kv_cache_scale_frames=1).to(dev, torch.bfloat16).eval()
    both = HipPagedKVCacheManager(1, 19, T, H, 64, torch.bfloat16, dev, num_special_tokens=5, scale_frames=1,
                                  sliding_window=2, max_total_frames=32, page_size=16, layout="frame_pages", num_streams=2)
    single = [HipPagedKVCacheManager(1, 19, T, H, 64, torch.bfloat16, dev, num_special_tokens=5, scale_frames=1,
                                     sliding_window=2, max_total_frames=32, page_size=16, layout="frame_pages")
              for _ in range(2)]
    with torch.no_grad():
        for f in range(6):
            x = torch.randn(2, T, dim, device=dev).to(torch.bfloat16)
            y = mod(x, kv_cache=both, global_idx=0, num_frames=1)
            for s in range(2):
                ys = mod(x[s:s + 1], kv_cache=single[s], global_idx=0, num_frames=1)
                assert (y[s:s + 1].float() - ys.float()).abs().max().item() <= 1e-2


@pytest.mark.parametrize("rope", ["none", "2d", "interleaved"])
def test_frame_block_without_cache_matches_torch_path(rope):
    """Cache-less frames (the aggregator's frame blocks): fused producer + paged kernel over a
    trivial row table against the same module's torch operations and SDPA in fp32."""
    import torch.nn.functional as F
    from lingbot_map_amd import HipPagedBlock, RotaryPositionEmbedding2D, dense_attention
    torch.manual_seed(8)
    dev = torch.device("cuda:0")
    dim, H, T, B = 256, 4, 333, 3
    mod = HipPagedBlock(dim, H, init_values=0.1, qk_norm=True,
                        rope={"none": None, "2d": RotaryPositionEmbedding2D(), "interleaved": True}[rope]).to(dev, torch.bfloat16).eval()
    for ln in (mod.attn.q_norm, mod.attn.k_norm):
        ln.weight.data.uniform_(0.5, 1.5)
        ln.bias.data.uniform_(-0.2, 0.2)
    x = torch.randn(B, T, dim, device=dev).to(torch.bfloat16)
    pos, e3 = None, False
    if rope == "2d":
        pos = torch.stack([torch.randint(0, 20, (1, T), device=dev), torch.randint(0, 20, (1, T), device=dev)], -1).expand(B, -1, -1).contiguous()
    if rope == "interleaved":
        ang = torch.rand(1, 1, T, 32, device=dev) * 6.283185
        pos, e3 = torch.polar(torch.ones_like(ang), ang), True
    with torch.no_grad():
        assert mod.attn.can_fuse_dense(mod.norm1(x), pos, e3)
        y = mod(x, pos=pos, enable_3d_rope=e3)
        q, k, v = mod.attn._qkv(mod.norm1(x), pos, e3)
        a = F.scaled_dot_product_attention(q.float(), k.float(), v.float()).transpose(1, 2).reshape(B, T, dim).to(torch.bfloat16)
        y_ref = mod.ffn_residual(x + mod.ls1(mod.attn.proj(a)))
        # the kernel alone, three independent groups in one launch
        nhd = lambda t: t.permute(0, 2, 1, 3).reshape(B * T, H, 64).contiguous()
        o = dense_attention(nhd(q), nhd(k), nhd(v), num_streams=B).reshape(B, T, dim)
    err = (o.float() - a.float()).abs()
    assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3
    err = (y.float() - y_ref.float()).abs()
    assert err.max().item() <= 3e-2 and err.mean().item() <= 2e-3


def test_camera_trunk_blocks_one_token_per_frame_fp32():
    """The camera head's trunk (lingbot_map/heads/camera_head.py:212-219, :296-346): blocks of 128-wide
    heads in fp32 over one camera token per frame at coordinates (f, 0, 0), the anchor frames in
    one call and every later frame on its own, nothing ever evicted (attention.py:307).  Checked
    against attention over the concatenation of every frame's K/V in float64."""
    from lingbot_map_amd import HipPagedBlock, HipPagedKVCacheManager, RotaryPositionEmbedding3D
    torch.manual_seed(9)
    dev = torch.device("cuda:0")
    dim, H, D, blocks, anchor, frames = 256, 2, 128, 4, 3, 45
    rope3d = RotaryPositionEmbedding3D(attention_head_dim=D, patch_size=(1024, 1, 1), fhw_dim=(40, 44, 44))
    mods = [HipPagedBlock(dim, H, init_values=0.5, qk_norm=True, rope=True, kv_cache_sliding_window=frames,
                          kv_cache_scale_frames=anchor).to(dev).eval() for _ in range(blocks)]
    m = HipPagedKVCacheManager(blocks, frames + 8, 1, H, D, torch.float32, dev, num_special_tokens=0,
                               scale_frames=anchor, sliding_window=frames, max_total_frames=frames + 8,
                               force_fp32=True, page_size=16, layout="frame_pages")
    seen_k = [[] for _ in range(blocks)]
    seen_v = [[] for _ in range(blocks)]
    f = 0
    with torch.no_grad():
        while f < frames:
            S = anchor if f == 0 else 1
            x = torch.randn(1, S, dim, device=dev)
            pos = rope3d(ppf=S, pph=1, ppw=1, patch_start_idx=0, device=dev, f_start=f, f_end=f + S)
            y, y_ref = x, x
            for b, mod in enumerate(mods):
                y = mod(y, pos=pos, enable_3d_rope=True, kv_cache=m, global_idx=b, num_frames=S)
                q, k, v = mod.attn_pre(y_ref, pos=pos, enable_3d_rope=True)      # [S, H, D]
                seen_k[b].append(k.double()); seen_v[b].append(v.double())
                K, V = torch.cat(seen_k[b]), torch.cat(seen_v[b])
                s = torch.einsum("qhd,khd->hqk", q.double(), K) / D ** 0.5
                a = torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), V).reshape(1, S, dim).float()
                y_ref = mod.ffn_residual(y_ref + mod.ls1(mod.attn.proj(a)))
            err = (y - y_ref).abs().max().item()
            assert err <= 2e-5, (f, err)
            f += S
    assert m.frame_count == [frames] * blocks and m.device_header()["error"] == 0


@pytest.mark.parametrize("reference_calls", [False, True])
def test_anchor_pass_over_several_frames_then_streaming(reference_calls):
    """Phase 1 of the streaming model (attention.py:475-511): the anchor frames arrive in one call,
    attend to one another densely, and are appended frame by frame, each block in turn, so block 0
    is several frames ahead of the others while they write.  Later frames stream one at a time
    and must see exactly the anchor frames and the window."""
    from lingbot_map_amd import HipPagedBlock, HipPagedKVCacheManager, keyframe_flags, set_skip_append
    from oracle.sdpa_cache import DictCacheOracle
    torch.manual_seed(11)
    dev = torch.device("cuda:0")
    dim, H, T, n_sp, scale, window, blocks = 256, 4, 37, 5, 3, 2, 3
    mods = [HipPagedBlock(dim, H, init_values=0.1, qk_norm=True, kv_cache_sliding_window=window,
                          kv_cache_scale_frames=scale).to(dev, torch.bfloat16).eval() for _ in range(blocks)]
    m = HipPagedKVCacheManager(blocks, scale + window + 16, T, H, 64, torch.bfloat16, dev, num_special_tokens=n_sp,
                               scale_frames=scale, sliding_window=window, max_total_frames=64, page_size=16,
                               layout="two_stream")
    cache = ReferenceSurfaceOnly(m) if reference_calls else m
    dense = [DictCacheOracle(scale, window, n_sp) for _ in range(blocks)]
    sdpa = lambda q, k, v: torch.nn.functional.scaled_dot_product_attention(
        q.float().permute(1, 0, 2)[None], k.float().permute(1, 0, 2)[None], v.float().permute(1, 0, 2)[None])[0].permute(1, 0, 2)
    flags = [True] * scale + keyframe_flags(9, 0, 2)
    with torch.no_grad():
        f = 0
        while f < len(flags):
            S = scale if f == 0 else 1
            kf = flags[f]
            x = torch.randn(1, S * T, dim, device=dev).to(torch.bfloat16)
            set_skip_append(cache, not kf)
            y, y_ref = x, x
            for b, mod in enumerate(mods):
                y = mod(y, kv_cache=cache, global_idx=b, num_frames=S)
                q, k, v = mod.attn_pre(y_ref)                                      # [S * T, H, D]
                if S > 1:
                    a = sdpa(q, k, v)
                    for i in range(S):
                        dense[b].visible(k[i * T:(i + 1) * T], v[i * T:(i + 1) * T], keyframe=True)
                else:
                    a = sdpa(q, *dense[b].visible(k, v, keyframe=kf))
                a = a.reshape(1, S * T, dim).to(torch.bfloat16)
                y_ref = mod.ffn_residual(y_ref + mod.ls1(mod.attn.proj(a)))
            set_skip_append(cache, False)
            err = (y.float() - y_ref.float()).abs()
            assert err.max().item() <= 3e-2 and err.mean().item() <= 2e-3, (f, err.max().item(), err.mean().item())
            f += S
    assert m.frame_count == [sum(flags)] * blocks and m.device_header()["error"] == 0 and not m._rows_log


def test_blocks_out_of_step_raise_with_shared_tables():
    """With one page table for all blocks a block may lag only while appending (the anchor pass);
    anything else out of step raises instead of reading or writing another frame's rows."""
    from lingbot_map_amd import HipPagedKVCacheManager
    dev = torch.device("cuda:0")
    H, D, T = 2, 64, 9
    mk = lambda **kw: HipPagedKVCacheManager(2, 24, T, H, D, torch.bfloat16, dev, num_special_tokens=1, scale_frames=1,
                                             sliding_window=2, max_total_frames=32, page_size=4, **kw)
    t = lambda: torch.randn(T, H, D, device=dev).to(torch.bfloat16)
    m = mk()
    with pytest.raises(RuntimeError, match="block 0 goes first"):
        m.append_frame(1, t(), t())
    m.append_frame(0, t(), t())
    assert m.compute_attention(1, t()).abs().max().item() == 0      # an empty block attends to nothing
    m.append_frame(0, t(), t())          # block 0 two frames ahead: allowed, rows of frame 0 are kept
    m.append_frame(1, t(), t())
    with pytest.raises(RuntimeError, match="compute_attention"):
        m.compute_attention(1, t())
    m.append_frame(1, t(), t())
    m.compute_attention(1, t())
    m.append_frame(0, t(), t())
    with pytest.raises(RuntimeError, match="block 0 starts a frame"):
        m.step(0, t(), t(), t())
    m.append_frame(1, t(), t())
    m.step(0, t(), t(), t())
    with pytest.raises(RuntimeError, match="block 0 goes first|no longer known"):
        m.append_frame(1, t(), t()); m.append_frame(1, t(), t())
    # per-block tables: any order
    p = mk(per_block_tables=True)
    p.append_frame(1, t(), t()); p.compute_attention(1, t()); p.append_frame(0, t(), t())
    assert p.device_header(0)["error"] == 0 and p.device_header(1)["error"] == 0


@pytest.mark.parametrize("rope", [False, True])
def test_chained_blocks_agree_with_the_separate_launches(rope):
    """Three blocks handing each other their row statistics (norm1 / norm2 folded into the qkv
    projection and fc1, proj / fc2 with LayerScale + residual in their store, lbm_linear_norm)
    against the same blocks run through the separate launches (LayerNorm + residual kernels,
    library GEMMs): streamed frames through a shared cache and a cache-less frame block.  The two
    paths round in different places, so the bar is the accumulated bf16 noise of three blocks, a
    small fraction of the activations' scale; the caches end up with the same page tables."""
    import math
    from lingbot_map_amd.block import HipPagedBlock, Mlp, RowStats, RotaryPositionEmbedding3D
    from lingbot_map_amd.manager import HipPagedKVCacheManager
    T, H, D, NS, frames = 70, 2, 64, 5, 4
    C = H * D
    torch.manual_seed(17)
    dev = torch.device("cuda:0")
    blocks = [HipPagedBlock(dim=C, num_heads=H, qk_norm=True, init_values=0.5, kv_cache_sliding_window=2, kv_cache_scale_frames=1,
                            rope=object() if rope else None).to(dev).to(torch.bfloat16).eval() for _ in range(3)]
    for b in blocks:
        for m in (b.norm1, b.norm2):
            m.weight.data.add_(0.2 * torch.randn_like(m.weight)); m.bias.data.add_(0.1 * torch.randn_like(m.bias))
    rope3d = RotaryPositionEmbedding3D(attention_head_dim=D, patch_size=(1, 14, 14), max_seq_len=64) if rope else None

    def manager():
        return HipPagedKVCacheManager(num_blocks=3, max_num_frames=6, tokens_per_frame=T, num_heads=H, head_dim=D,
                                      dtype=torch.bfloat16, device=dev, num_special_tokens=NS, scale_frames=1, sliding_window=2,
                                      max_total_frames=32)

    def run(chained: bool):
        limit = Mlp.FUSED_MAX_ROWS
        Mlp.FUSED_MAX_ROWS = limit if chained else 0     # no fused launch qualifies: the separate ones run
        try:
            m, outs, kinds = manager(), [], []
            for f in range(frames):
                x = torch.randn(1, T, C, generator=torch.Generator().manual_seed(100 + f)).to(dev).to(torch.bfloat16)
                pos = rope3d(ppf=1, pph=5, ppw=13, patch_start_idx=NS, device=dev, f_start=f, f_end=f + 1) if rope else None
                normed = None
                with torch.no_grad():
                    for i, b in enumerate(blocks):
                        nxt = blocks[i + 1].norm1 if i + 1 < len(blocks) else None
                        r = b(x, pos=pos, kv_cache=m, global_idx=i, enable_3d_rope=rope, normed=normed, next_norm=nxt,
                              num_frames=1, num_register_tokens=NS - 1)
                        x, normed = r if nxt is not None else (r, None)
                        kinds.append(type(normed).__name__)
                outs.append(x.float().cpu())
            tables = [m.build_visible_page_table(i) for i in range(3)]
            return outs, kinds, tables
        finally:
            Mlp.FUSED_MAX_ROWS = limit

    got, kinds, tables = run(True)
    ref, ref_kinds, ref_tables = run(False)
    assert "RowStats" in kinds and "RowStats" not in ref_kinds       # the chain really ran, and only there
    assert tables == ref_tables
    for a, b in zip(got, ref):
        assert torch.isfinite(a).all()
        scale = b.abs().mean().item()
        assert (a - b).abs().mean().item() <= 0.01 * scale, ((a - b).abs().mean().item(), scale)
        assert (a - b).abs().max().item() <= 0.1 * max(scale, 1.0)
    # a frame block (no cache) fed with statistics, against the same block fed with norm1(x)
    blk = HipPagedBlock(dim=C, num_heads=H, qk_norm=True, init_values=0.5).to(dev).to(torch.bfloat16).eval()
    x = torch.randn(2, T, C, generator=torch.Generator().manual_seed(5)).to(dev).to(torch.bfloat16)
    with torch.no_grad():
        lin = torch.nn.Linear(C, C).to(dev).to(torch.bfloat16)
        x0 = torch.randn_like(x)
        # statistics of x as a residual launch leaves them: x = x0 + lin(h) recomputed through the chain's own helper
        xr, st = blk._linear_residual(x0, lin, torch.nn.Identity(), x0, True)
        y_stats, _ = blk(xr, normed=st, next_norm=blocks[1].norm1)
        y_norm, _ = blk(xr, normed=blk.norm1(xr), next_norm=blocks[1].norm1)
    assert isinstance(st, RowStats)
    d = (y_stats.float() - y_norm.float()).abs()
    assert d.mean().item() <= 0.01 * y_norm.float().abs().mean().item()
