"""The streaming aggregator shell (lingbot_map_amd/aggregator.py) on the GPU.

1. Reduced depth and width, two ragged streams, keyframes and non-keyframes: every group's
   output against the same weights evaluated in fp32 torch on the CPU - special tokens first,
   frame block then global block, 2-D rotary embedding in the frame blocks and the 3-D table in
   the global blocks, the dict-cache semantics of the reference's SDPA path (DictCacheOracle)
   per block and stream.  fp32 cache: max-abs 1e-4.  bf16: the 2e-2 / 2e-3 bars belong to the
   attention output alone; here that output passes through the projection, LayerScale 1 and the
   MLP of every later block and the compared activations reach magnitudes of several units, so
   the bars are relative: max-abs <= 2 % of the largest and mean-abs <= 1 % of the mean
   magnitude of the fp32 result.
2. Configuration 5 at full depth and width: 24 groups, four streams with windows 4/8/16/16,
   1004 tokens per frame; page tables of every stream bit-exact against the page policy after
   every frame, outputs finite."""
import math

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def f32(t):
    return t.detach().float().cpu()


def ln(x, m):
    return F.layer_norm(x, (x.shape[-1],), f32(m.weight), f32(m.bias), m.eps)


class TorchReference:
    """fp32 CPU evaluation of a HipAggregatorStream's weights, one streamed frame per call."""

    def __init__(self, model, windows, anchor):
        from oracle.sdpa_cache import DictCacheOracle
        self.m = model
        self.caches = [[DictCacheOracle(anchor, w, model.num_special_tokens, model.kv_cache_cross_frame_special,
                                        True, model.kv_cache_camera_only) for w in windows]
                       for _ in range(model.depth)]
        self.cached_frames = 0       # frames in the cache (keyframes)
        self.streamed_frames = 0     # frames whose index the 3-D table has used

    def special_tokens(self, B, S):
        # stream.py:336-357: expand for every frame so far, index 0 of each pair for the first
        # frame (scale token: the first num_frame_for_scale frames), keep the current frames
        m = self.m
        total = self.cached_frames + S
        first = lambda tok, n: torch.cat([f32(tok)[:, :1].expand(1, n, -1, -1), f32(tok)[:, 1:].expand(1, total - n, -1, -1)], 1)
        parts = [first(m.camera_token, 1)]
        if m.num_register_tokens:
            parts.append(first(m.register_token, 1))
        if m.use_scale_token:
            parts.append(first(m.scale_token, max(min(m.num_frame_for_scale, total), 1)))
        tok = torch.cat(parts, dim=2)[0, -S:]                       # [S, n, C]
        return tok.unsqueeze(0).expand(B, -1, -1, -1).reshape(B * S, tok.shape[1], -1)

    def block(self, blk, x, rotate, attend):
        N, P, C = x.shape
        Hh, D = blk.attn.num_heads, blk.attn.head_dim
        h = ln(x, blk.norm1)
        qkv = F.linear(h, f32(blk.attn.qkv.weight), f32(blk.attn.qkv.bias)).reshape(N, P, 3, Hh, D).permute(2, 0, 3, 1, 4)
        q, k, v = qkv.unbind(0)                                       # [N, H, P, D]
        q, k = ln(q, blk.attn.q_norm), ln(k, blk.attn.k_norm)
        q, k = rotate(q), rotate(k)
        o = attend(q, k, v)                                           # [N, P, H * D]
        x = x + f32(blk.ls1.gamma) * F.linear(o, f32(blk.attn.proj.weight), f32(blk.attn.proj.bias))
        h = ln(x, blk.norm2)
        h = F.linear(F.gelu(F.linear(h, f32(blk.mlp.fc1.weight), f32(blk.mlp.fc1.bias))),
                     f32(blk.mlp.fc2.weight), f32(blk.mlp.fc2.bias))
        return x + f32(blk.ls2.gamma) * h

    def step(self, images, keyframe):
        from oracle.prepare_qkv import apply_rotary_emb, rope2d, rope3d_freqs
        from oracle.sdpa_cache import sdpa_nhd
        m = self.m
        B, S, _, H, W = images.shape
        assert S == 1
        x = (images.float().cpu() - torch.tensor([0.485, 0.456, 0.406]).view(1, 1, 3, 1, 1)) / \
            torch.tensor([0.229, 0.224, 0.225]).view(1, 1, 3, 1, 1)
        patches = F.conv2d(x.view(B * S, 3, H, W), f32(m.patch_embed.proj.weight), f32(m.patch_embed.proj.bias),
                           stride=m.patch_size).flatten(2).transpose(1, 2)
        tokens = torch.cat([self.special_tokens(B, S), patches], dim=1)
        P = tokens.shape[1]
        gh, gw = H // m.patch_size, W // m.patch_size
        ys, xs = torch.meshgrid(torch.arange(gh), torch.arange(gw), indexing="ij")
        grid = torch.stack([ys.reshape(-1), xs.reshape(-1)], -1) + 1
        pos = torch.cat([torch.zeros(m.num_special_tokens, 2, dtype=torch.long), grid])[None].expand(B * S, -1, -1)
        freqs = rope3d_freqs(ppf=1, pph=gh, ppw=gw, patch_start_idx=m.num_special_tokens,
                             head_dim=m.embed_dim // m.num_heads, max_seq_len=m.max_frame_num,
                             f_start=self.streamed_frames, f_end=self.streamed_frames + 1)
        outs = []
        for g in range(m.depth):
            tokens = self.block(m.frame_blocks[g], tokens, lambda t: rope2d(t, pos),
                                lambda q, k, v: F.scaled_dot_product_attention(q, k, v).transpose(1, 2).reshape(B * S, P, -1))
            frame_out = tokens

            def attend(q, k, v, g=g):
                rows = []
                for b in range(B):
                    nhd = lambda t: t[b].permute(1, 0, 2).contiguous()
                    rows.append(self.caches[g][b].step(nhd(q), nhd(k), nhd(v), keyframe=keyframe).reshape(P, -1))
                return torch.stack(rows)
            tokens = self.block(m.global_blocks[g], tokens, lambda t: apply_rotary_emb(t, freqs.to(torch.complex64)), attend)
            outs.append(torch.cat([frame_out, tokens], dim=-1).view(B, S, P, -1))
        if keyframe:
            self.cached_frames += 1
            self.streamed_frames += 1
        return outs


@pytest.mark.parametrize("dtype,bar", [(torch.float32, 1e-4), (torch.bfloat16, None)])
def test_aggregator_matches_fp32_torch_with_dict_caches(dtype, bar):
    from lingbot_map_amd import HipAggregatorStream, set_skip_append
    dev = torch.device("cuda:0")
    torch.manual_seed(5)
    windows, anchor = [2, 3], 1
    model = HipAggregatorStream(img_size=56, patch_size=14, embed_dim=128, depth=2, num_heads=2, init_values=1.0,
                                patch_embed="conv", enable_3d_rope=True, max_frame_num=64,
                                kv_cache_sliding_window=windows, kv_cache_scale_frames=anchor,
                                kv_cache_force_fp32=dtype == torch.float32, use_scale_token=False, page_size=4,
                                layout="frame_pages", num_streams=2)
    with torch.no_grad():
        for tok in (model.camera_token, model.register_token):
            tok.normal_(std=1.0)
        for blk in list(model.frame_blocks) + list(model.global_blocks):   # LayerNorms off their identity init
            for norm in (blk.norm1, blk.norm2, blk.attn.q_norm, blk.attn.k_norm):
                norm.weight.uniform_(0.5, 1.5)
                norm.bias.uniform_(-0.2, 0.2)
    model = model.to(dev).eval()
    ref = TorchReference(model, windows, anchor)      # reads the fp32 master weights
    if dtype == torch.bfloat16:
        model = model.to(torch.bfloat16)
    assert model.num_special_tokens == 5 and model.patch_start_idx == 5
    g = torch.Generator().manual_seed(6)
    pattern = [True, True, False, True, False, False, True, True, True, False, True]
    with torch.no_grad():
        for f, keyframe in enumerate(pattern):
            images = torch.rand(2, 1, 3, 42, 56, generator=g)
            want = ref.step(images, keyframe)
            set_skip_append(model._get_manager(dev, dtype, 17), not keyframe)
            got, start = model(images.to(dev, dtype))
            assert start == 5 and len(got) == 2
            for a, b in zip(got, want):
                assert a.shape == b.shape == (2, 1, 17, 256)
                err = (a.float().cpu() - b).abs()
                if bar is not None:
                    assert err.max().item() <= bar, (f, keyframe, err.max().item())
                else:
                    assert err.max().item() <= 0.02 * b.abs().max().item(), (f, keyframe, err.max().item(), b.abs().max().item())
                    assert err.mean().item() <= 0.01 * b.abs().mean().item(), (f, keyframe, err.mean().item(), b.abs().mean().item())
    mgr = model.kv_cache_manager
    assert mgr.num_frames == sum(pattern) and model.total_frames_processed == sum(pattern)
    assert mgr.get_cache_stats(0, stream=0)["live_pages"] == 2 * mgr.pages_per_frame
    assert mgr.get_cache_stats(0, stream=1)["live_pages"] == 3 * mgr.pages_per_frame
    mgr.check_device_errors()
    model.clean_kv_cache()
    assert mgr.num_frames == 0 and model.total_frames_processed == 0


def test_config5_full_depth_four_ragged_streams():
    from lingbot_map_amd import HipAggregatorStream
    from oracle.page_policy import PagePolicy
    dev = torch.device("cuda:0")
    torch.manual_seed(4)
    windows, anchor, T = [4, 8, 16, 16], 1, 1004
    model = HipAggregatorStream(img_size=518, patch_size=14, embed_dim=1024, depth=24, num_heads=16, patch_embed="conv",
                                enable_3d_rope=True, max_frame_num=156, kv_cache_sliding_window=windows,
                                kv_cache_scale_frames=anchor, use_scale_token=False, page_size=16, layout="frame_pages",
                                num_streams=4).to(dev, torch.bfloat16).eval()
    g = torch.Generator(device=dev).manual_seed(4)
    pols = None
    with torch.no_grad():
        for f in range(20):
            images = torch.rand(4, 1, 3, 378, 518, generator=g, device=dev).to(torch.bfloat16)
            outs, start = model(images, selected_idx=[4, 11, 17, 23])
            assert start == 5 and len(outs) == 4 and outs[-1].shape == (4, 1, T, 2048)
            assert all(torch.isfinite(o.float()).all() for o in outs), f
            mgr = model.kv_cache_manager
            if pols is None:
                assert mgr.tokens_per_frame == T and mgr.num_blocks == 24 and mgr.num_streams == 4
                pols = [PagePolicy(T, 5, 16, anchor, 16, 256, layout="frame_pages", page_base=b * mgr.max_num_pages)
                        for b in range(4)]
                assert all(p.max_num_pages == mgr.max_num_pages for p in pols)
            for b in range(4):
                pols[b].append_frame()
                pols[b].evict_frames(anchor, windows[b])
                assert mgr.build_visible_page_table(0, stream=b) == pols[b].build_visible_page_table(), (f, b)
                assert mgr.build_visible_page_lens(0, stream=b) == pols[b].build_visible_page_lens(), (f, b)
    for b in range(4):
        assert pols[b].visible_tokens() == (anchor + windows[b]) * T + 5 * (20 - anchor - windows[b])
        assert mgr.get_cache_stats(23, stream=b) == pols[b].get_cache_stats()
    assert mgr.frame_count == [20] * 24 and model.total_frames_processed == 20
    mgr.check_device_errors()


def test_full_width_single_stream_against_fp32_torch():
    """The width the model ships at - dim 1024, 16 heads, MLP 4096, 1004 tokens per 378 x 518
    frame - at depth 2, one stream: the path on which every linear is the package's GEMM with the
    LayerNorms folded in, GELU, LayerScale + residual and the producer in its stores.  Three
    streamed frames (two keyframes and a read-only one) against the same weights in fp32 torch on
    the CPU with dict caches; relative bars as above."""
    from lingbot_map_amd import HipAggregatorStream, set_skip_append
    dev = torch.device("cuda:0")
    torch.manual_seed(9)
    windows, anchor = [16], 1
    model = HipAggregatorStream(img_size=518, patch_size=14, embed_dim=1024, depth=2, num_heads=16, init_values=1.0,
                                patch_embed="conv", enable_3d_rope=True, max_frame_num=64,
                                kv_cache_sliding_window=windows, kv_cache_scale_frames=anchor, use_scale_token=False,
                                page_size=16, layout="frame_pages", num_streams=1)
    with torch.no_grad():
        for tok in (model.camera_token, model.register_token):
            tok.normal_(std=1.0)
        for blk in list(model.frame_blocks) + list(model.global_blocks):
            for norm in (blk.norm1, blk.norm2, blk.attn.q_norm, blk.attn.k_norm):
                norm.weight.uniform_(0.5, 1.5)
                norm.bias.uniform_(-0.2, 0.2)
    model = model.to(dev).eval()
    ref = TorchReference(model, windows, anchor)
    model = model.to(torch.bfloat16)
    g = torch.Generator().manual_seed(10)
    with torch.no_grad():
        for f, keyframe in enumerate([True, True, False]):
            images = torch.rand(1, 1, 3, 378, 518, generator=g)
            want = ref.step(images, keyframe)
            set_skip_append(model._get_manager(dev, torch.bfloat16, 1004), not keyframe)
            got, start = model(images.to(dev, torch.bfloat16))
            assert start == 5 and len(got) == 2
            for a, b in zip(got, want):
                assert a.shape == b.shape == (1, 1, 1004, 2048)
                err = (a.float().cpu() - b).abs()
                assert err.max().item() <= 0.02 * b.abs().max().item(), (f, keyframe, err.max().item(), b.abs().max().item())
                assert err.mean().item() <= 0.01 * b.abs().mean().item(), (f, keyframe, err.mean().item(), b.abs().mean().item())
    model.kv_cache_manager.check_device_errors()
