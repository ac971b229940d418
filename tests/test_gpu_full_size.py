"""The benchmark configurations at their FULL sizes against the CPU oracle (GPU).

config 2  200 streamed steps at 1004 tokens x 16 heads, page 16, 1 anchor + 16 window frames:
          page tables bit-exact after every step, attention outputs every 40 steps
config 3  the state a 10,000-frame stream ends in: 1004 anchor + 16,064 window + 49,915 memory
          tokens = 66,983 visible tokens over 11,054 pages (the 67,068 of the configuration text counts all
          10,000 frames as evicted), native order and seed-2 shuffled page-table order
config 4  72 frames at full frame size, keyframe interval 4: tables after every step, pool
          untouched by non-keyframes, outputs on keyframes and non-keyframes

Tolerances: page ids, lengths and counts bit-exact; bf16 outputs max-abs <= 2e-2 and mean-abs
<= 2e-3 against fp32 SDPA on the same bf16 inputs, and - because N(0,1) values averaged over
17,000+ tokens are small - also mean-abs <= 1 % of the mean magnitude of the reference."""
import ctypes as C
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

BF16_MAX_ABS, BF16_MEAN_ABS, REL_MEAN = 2e-2, 2e-3, 0.01
T, H, D, S, N_SP, ANCHOR, WINDOW = 1004, 16, 64, 16, 5, 1, 16


def manager(**kw):
    from lingbot_map_amd import HipPagedKVCacheManager
    args = dict(num_blocks=1, max_num_frames=ANCHOR + WINDOW + 16, tokens_per_frame=T, num_heads=H, head_dim=D,
                dtype=torch.bfloat16, device=torch.device("cuda:0"), num_special_tokens=N_SP, scale_frames=ANCHOR,
                sliding_window=WINDOW, max_total_frames=256, page_size=S, layout="frame_pages")
    args.update(kw)
    return HipPagedKVCacheManager(**args)


def check(out, ref, what):
    err = (out.float().cpu() - ref.float()).abs()
    assert torch.isfinite(out.float()).all(), what
    assert err.max().item() <= BF16_MAX_ABS, (what, err.max().item())
    assert err.mean().item() <= BF16_MEAN_ABS, (what, err.mean().item())
    assert err.mean().item() <= REL_MEAN * ref.float().abs().mean().item(), (what, err.mean().item(), ref.float().abs().mean().item())


def test_config2_two_hundred_streamed_steps_full_size():
    from oracle.page_policy import PagePolicy
    from oracle.sdpa_cache import PagedStreamOracle
    m = manager()
    pol = PagePolicy(T, N_SP, S, ANCHOR, WINDOW, 256, layout="frame_pages")
    orc = PagedStreamOracle(pol, H, D, torch.bfloat16)
    g = torch.Generator().manual_seed(1)
    checked = 0
    for step in range(200):
        q, k, v = (torch.randn(T, H, D, generator=g).to(torch.bfloat16) for _ in range(3))
        # evicted frames leave no trajectory memory: the KV set stays at 17 frames = 17,068 tokens
        out = m.step(0, q.cuda(), k.cuda(), v.cuda(), keyframe=[True], cross_frame_special=False)
        orc.append_frame(k, v)
        pol.evict_frames(ANCHOR, WINDOW, cross_frame_special=False)
        assert m.build_visible_page_table(0) == pol.build_visible_page_table(), step
        assert m.build_visible_page_lens(0) == pol.build_visible_page_lens(), step
        if step % 40 == 39 or step in (0, 16, 17):
            check(out, orc.compute_attention(q), f"step {step}")
            checked += 1
    assert checked == 8 and pol.visible_tokens() == 17068 == (ANCHOR + WINDOW) * T
    assert m.get_cache_stats() == pol.get_cache_stats()
    m.check_device_errors()


def test_config4_full_frame_size_keyframe_interval_four():
    from oracle.page_policy import PagePolicy, is_keyframe
    from oracle.sdpa_cache import PagedStreamOracle
    frames = 72
    m = manager()
    pol = PagePolicy(T, N_SP, S, ANCHOR, WINDOW, 256, layout="frame_pages")
    orc = PagedStreamOracle(pol, H, D, torch.bfloat16)
    g = torch.Generator().manual_seed(3)
    appended = 0
    for f in range(frames):
        kf = is_keyframe(f, ANCHOR, 4)
        appended += kf
        q, k, v = (torch.randn(T, H, D, generator=g).to(torch.bfloat16) for _ in range(3))
        compare = f in (0, 1, 2, 4, 5, 33, 64, 65, 66, 67, 68, 69, 70, 71)
        if kf:
            orc.append_frame(k, v)
            pol.evict_frames(ANCHOR, WINDOW)
            ref = orc.compute_attention(q) if compare else None
        else:
            ref = orc.step(q, k, v, keyframe=False) if compare else None   # append, attend, roll back
            tables_before, pool_before = m._tables.clone(), m.kv_caches[0].clone()
        out = m.step(0, q.cuda(), k.cuda(), v.cuda(), keyframe=[kf])
        if not kf:    # every table word but the plan's own two and every pool byte stay as they were
            assert torch.equal(m._tables[..., :11], tables_before[..., :11]), f
            assert torch.equal(m.kv_caches[0], pool_before), f
        if compare:
            check(out, ref, f"frame {f} keyframe={kf}")
        assert m.build_visible_page_table(0) == pol.build_visible_page_table(), f
        assert m.build_visible_page_lens(0) == pol.build_visible_page_lens(), f
    # 1 anchor + 18 keyframes appended, two of them already compacted to their 5 memory tokens
    assert appended == 19 and m.frame_count[0] == 19 and m.get_cache_stats() == pol.get_cache_stats()
    assert pol.visible_tokens() == 17 * T + 2 * N_SP
    m.check_device_errors()


def test_config3_end_of_ten_thousand_frame_stream_full_size():
    """All 10,000 frames are appended at full size on the GPU (K/V generated there).  The oracle
    gets, of every frame, what can still be visible at the end - the page with its leading
    special tokens - and the anchor and the last 16 frames in full."""
    from lingbot_map_amd import _native as N
    from oracle.page_policy import PagePolicy
    from oracle.sdpa_cache import PagedStreamOracle, write_frame
    frames = 10000
    dev = torch.device("cuda:0")
    m = manager(max_total_frames=frames)
    pol = PagePolicy(T, N_SP, S, ANCHOR, WINDOW, frames, layout="frame_pages")
    assert m.max_num_pages == pol.max_num_pages
    orc = PagedStreamOracle(pol, H, D, torch.bfloat16)
    g = torch.Generator(device=dev).manual_seed(2)
    # eight distinct frames of K/V, cycled with a per-frame sign/scale so that no two frames agree
    base = [torch.randn(2, T, H, D, generator=g, device=dev).to(torch.bfloat16) for _ in range(8)]
    base_cpu = [b.cpu() for b in base]
    head_rows = S    # tokens of a frame's first page
    for f in range(frames):
        scale = 1.0 if (f // 8) % 2 == 0 else -1.0
        kv = base[f % 8] * scale
        m.append_frame(0, kv[0], kv[1])
        m.evict_frames(0, ANCHOR, WINDOW)
        plan = pol.append_frame()
        pol.evict_frames(ANCHOR, WINDOW)
        full = f < ANCHOR or f >= frames - WINDOW
        n = T if full else head_rows
        kc = base_cpu[f % 8][:, :n] * scale
        write_frame(orc.pool, plan.page[:n], plan.slot[:n], kc[0], kc[1])
        if f in (17, 18, 4999):
            assert m.build_visible_page_table(0) == pol.build_visible_page_table(), f
    ids, lens = m.build_visible_page_table(0), m.build_visible_page_lens(0)
    assert ids == pol.build_visible_page_table() and lens == pol.build_visible_page_lens()
    n_mem = frames - ANCHOR - WINDOW
    n_tok = (ANCHOR + WINDOW) * T + N_SP * n_mem
    assert sum(lens) == n_tok == 66983 and len(ids) == (ANCHOR + WINDOW) * 63 + n_mem == 11054
    assert lens[-n_mem:] == [N_SP] * n_mem
    assert m.get_cache_stats() == pol.get_cache_stats()
    # every memory page holds 5 live tokens in 16 slots, and no page id appears twice
    assert len(set(ids)) == len(ids)
    q = torch.randn(T, H, D, generator=g, device=dev).to(torch.bfloat16)
    ref = orc.compute_attention(q.cpu())
    # native order, through the manager
    check(m.compute_attention(0, q), ref, "native order")
    # page-table order shuffled with seed 2, through the general entry points
    perm = torch.randperm(len(ids), generator=torch.Generator().manual_seed(2)).tolist()
    ids_d = torch.tensor([ids[i] for i in perm], dtype=torch.int32, device=dev)
    lens_d = torch.tensor([lens[i] for i in perm], dtype=torch.int32, device=dev)
    rows = torch.empty(n_tok, dtype=torch.int32, device=dev)
    i32 = C.c_int32
    p = lambda t: C.c_void_p(t.data_ptr())
    N.check(N.lib.lbm_rows_from_pages(p(ids_d), p(lens_d), (i32 * 2)(0, len(ids)), (i32 * 1)(n_tok), (i32 * 1)(0),
                                      1, S, p(rows), None))
    st = (N.AttnStream * 1)(N.AttnStream(0, T, 0, n_tok))
    need = int(N.lib.lbm_attn_workspace_bytes(st, 1, H, D))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    out = torch.full_like(q, float("nan"))
    N.check(N.lib.lbm_attn_run(p(q), p(m.kv_caches[0]), p(out), None, None, p(rows), st, 1, H, D, S,
                               N.DTYPE_BF16, 1.0 / math.sqrt(D), p(ws), ws.numel(), None))
    torch.cuda.synchronize()
    check(out, ref, "shuffled order")
    m.check_device_errors()


def test_config5_four_ragged_streams_in_one_launch():
    """Configuration 5's attention launch by itself, at full size: four streams of 1004 query rows
    with 5,020 / 9,036 / 17,068 / 17,068 visible tokens (windows 4 / 8 / 16 / 16 plus the anchor
    frame) in ONE ``lbm_attn_run``, pages in shuffled order, seed 4; every stream against the
    oracle's SDPA on its own tokens, with the relative bar as well."""
    from lingbot_map_amd import _native as N
    from oracle.sdpa_cache import gather_paged, sdpa_nhd
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(4)
    kv_tokens = [(1 + w) * T for w in (4, 8, 16, 16)]
    assert kv_tokens == [5020, 9036, 17068, 17068]
    pages_per_frame = (T + S - 1) // S                       # 63: 62 full pages and one of 12 tokens
    n_pages = sum(n // T for n in kv_tokens) * pages_per_frame
    pool = torch.randn(n_pages, 2, S, H, D, generator=g).to(torch.bfloat16)
    q = torch.randn(4 * T, H, D, generator=g).to(torch.bfloat16)
    order = torch.randperm(n_pages, generator=g).tolist()
    ids, lens, indptr, at = [], [], [0], 0
    for n in kv_tokens:
        for _ in range(n // T):
            ids += order[at:at + pages_per_frame]
            lens += [S] * (pages_per_frame - 1) + [T - S * (pages_per_frame - 1)]
            at += pages_per_frame
        indptr.append(len(ids))
    i32 = C.c_int32
    row_begin = [sum(kv_tokens[:b]) for b in range(4)]
    ids_d, lens_d = torch.tensor(ids, dtype=torch.int32, device=dev), torch.tensor(lens, dtype=torch.int32, device=dev)
    rows = torch.empty(sum(kv_tokens), dtype=torch.int32, device=dev)
    ptr = lambda t: C.c_void_p(t.data_ptr())
    N.check(N.lib.lbm_rows_from_pages(ptr(ids_d), ptr(lens_d), (i32 * 5)(*indptr), (i32 * 4)(*kv_tokens), (i32 * 4)(*row_begin),
                                      4, S, ptr(rows), None))
    streams = (N.AttnStream * 4)(*[N.AttnStream(b * T, T, row_begin[b], kv_tokens[b]) for b in range(4)])
    ws = torch.empty(max(int(N.lib.lbm_attn_workspace_bytes(streams, 4, H, D)), 16), dtype=torch.uint8, device=dev)
    qd, pd = q.to(dev), pool.to(dev)
    out = torch.full_like(qd, float("nan"))
    N.check(N.lib.lbm_attn_run(ptr(qd), ptr(pd), ptr(out), None, None, ptr(rows), streams, 4, H, D, S, N.DTYPE_BF16,
                               1.0 / math.sqrt(D), ptr(ws), ws.numel(), None))
    torch.cuda.synchronize()
    for b in range(4):
        kk, vv = gather_paged(pool, ids[indptr[b]:indptr[b + 1]], lens[indptr[b]:indptr[b + 1]])
        assert kk.shape[0] == kv_tokens[b]
        check(out[b * T:(b + 1) * T], sdpa_nhd(q[b * T:(b + 1) * T], kk, vv), f"stream {b}: {kv_tokens[b]} tokens")


@pytest.mark.parametrize("n_streams", [1, 2, 4])
def test_frame_blocks_of_several_streams_at_full_size(n_streams):
    """The frame and encoder blocks' cache-less attention (``dense_attention``: 1004 x 1004 per
    stream, 16 heads) for one, two and four streams in one launch.  The schedule prices the
    short-KV kernel against the split-KV pair: one and two streams take the short-KV kernel (no
    workspace), four streams - four rounds of the CUs on the short-KV kernel - take the pair.
    Either way every stream must match the oracle's SDPA on its own tokens."""
    from lingbot_map_amd import _native as N, dense_attention
    from oracle.sdpa_cache import sdpa_nhd
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(20 + n_streams)
    q, k, v = (torch.randn(n_streams * T, H, D, generator=g).to(torch.bfloat16) for _ in range(3))
    streams = (N.AttnStream * n_streams)(*[N.AttnStream(s * T, T, s * T, T) for s in range(n_streams)])
    need = int(N.lib.lbm_attn_workspace_bytes(streams, n_streams, H, D))
    assert (need > 0) == (n_streams == 4), (n_streams, need)
    out = dense_attention(q.to(dev), k.to(dev), v.to(dev), num_streams=n_streams).cpu()
    for s in range(n_streams):
        sl = slice(s * T, (s + 1) * T)
        check(out[sl], sdpa_nhd(q[sl], k[sl], v[sl]), f"stream {s} of {n_streams}")


@pytest.mark.parametrize("n_streams", [1, 2])
def test_lookahead_replay_at_full_width(n_streams):
    """The look-ahead replay (next frame's encoder beside the present frame's blocks) at the real
    widths - 1,004 tokens per frame, dim 1,024, MLP 4,096, so that fc2 splits K over workgroups in
    both branches (each on the workspace of its own scratch lane) and the launches of the two
    branches share the CUs - against the plain replay of a twin model: bit-equal outputs, frame by
    frame, and equal pools."""
    from lingbot_map_amd import GraphedAggregator, HipAggregatorStream, PipelinedAggregator
    dev = torch.device("cuda:0")
    kw = dict(img_size=518, patch_size=14, embed_dim=1024, depth=3, num_heads=16, mlp_ratio=4.0, num_register_tokens=4,
              qk_norm=True, init_values=0.01, patch_embed="vit", encoder_depth=3, enable_3d_rope=True, max_frame_num=64,
              kv_cache_sliding_window=[3, 2][:n_streams] if n_streams > 1 else 3, kv_cache_scale_frames=1,
              kv_cache_cross_frame_special=False, use_scale_token=False, page_size=16, layout="frame_pages",
              num_streams=n_streams)
    torch.manual_seed(21)
    a = HipAggregatorStream(**kw).to(dev, torch.bfloat16).eval()
    b = HipAggregatorStream(**kw).to(dev, torch.bfloat16).eval()
    b.load_state_dict(a.state_dict())
    g = torch.Generator(device=dev).manual_seed(22)
    imgs = [torch.rand(n_streams, 1, 3, 378, 518, generator=g, device=dev).to(torch.bfloat16) for _ in range(4)]
    with torch.no_grad():
        for i in range(5):                       # anchor and windows full
            a(imgs[i % 4]); b(imgs[i % 4])
        plain = GraphedAggregator(a, imgs[0])
        piped = PipelinedAggregator(b, imgs[0])
        frames = [imgs[(3 * i + 1) % 4] for i in range(8)]
        piped.prime(frames[0])
        for i in range(7):
            keyframe = i % 4 != 2
            want = plain(frames[i], keyframe=keyframe).clone()
            got = piped(frames[i + 1], keyframe=keyframe)
            torch.cuda.synchronize()
            assert torch.isfinite(got.float()).all()
            assert torch.equal(got, want), (i, keyframe)
    for x, y in zip(a.kv_cache_manager.kv_caches, b.kv_cache_manager.kv_caches):
        assert torch.equal(x, y)
    b.kv_cache_manager.check_device_errors()
