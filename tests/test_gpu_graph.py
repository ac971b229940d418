"""A steady-state streamed frame captured as a HIP graph replays to the same results as the
eager path: outputs bit for bit on every replay (with eager work and synchronisations in
between), device page tables and pools identical afterwards."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _setup(cross_frame_special, device_token_counts=False):
    from lingbot_map_amd import HipPagedBlock, HipPagedKVCacheManager, RotaryPositionEmbedding2D
    torch.manual_seed(12)
    dev = torch.device("cuda:0")
    dim, H, T, blocks, scale, window = 256, 4, 53, 2, 1, 3
    kw = dict(dim=dim, num_heads=H, qk_norm=True, init_values=0.1, kv_cache_sliding_window=window,
              kv_cache_scale_frames=scale, kv_cache_cross_frame_special=cross_frame_special)
    rope2d = RotaryPositionEmbedding2D()
    fb = [HipPagedBlock(rope=rope2d, **kw).to(dev, torch.bfloat16).eval() for _ in range(blocks)]
    gb = [HipPagedBlock(rope=True, **kw).to(dev, torch.bfloat16).eval() for _ in range(blocks)]
    mk = lambda: HipPagedKVCacheManager(blocks, scale + window + 16, T, H, 64, torch.bfloat16, dev, num_special_tokens=5,
                                        scale_frames=scale, sliding_window=window, max_total_frames=64, page_size=16,
                                        layout="frame_pages", device_token_counts=device_token_counts)
    ang = torch.rand(1, 1, T, 32, device=dev) * 6.283185
    freqs = torch.polar(torch.ones_like(ang), ang)
    pos2d = torch.stack([torch.randint(0, 9, (1, T), device=dev), torch.randint(0, 9, (1, T), device=dev)], -1)

    def frame_on(m):
        @torch.no_grad()
        def frame(x):
            for b in range(blocks):
                x = fb[b](x, pos=pos2d)
                x = gb[b](x, pos=freqs, enable_3d_rope=True, kv_cache=m, global_idx=b)
            return x
        return frame

    xs = [torch.randn(1, T, dim, device=dev).to(torch.bfloat16) for _ in range(6)]
    return mk, frame_on, xs, scale + window


def test_graph_replay_equals_eager():
    from lingbot_map_amd import GraphedFrame
    mk, frame_on, xs, fill = _setup(cross_frame_special=False)
    eager, graphed = mk(), mk()
    f_e, f_g = frame_on(eager), frame_on(graphed)
    assert not graphed.steady_state(cross_frame_special=False)
    for i in range(fill + 2):
        f_e(xs[i % 6]); f_g(xs[i % 6])
    assert graphed.steady_state(cross_frame_special=False)
    before = graphed._tables.clone()
    g = GraphedFrame(graphed, f_g, [xs[0]], cross_frame_special=False)   # warm-up and capture leave the cache alone
    assert torch.equal(graphed._tables[..., :11], before[..., :11])
    assert graphed.frame_count == eager.frame_count
    for i in range(8):
        x = xs[(3 * i + 1) % 6]
        want = f_e(x)
        got = g(x)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {i}"
        # the program's own eager work between replays
        _ = (torch.randn(256, 256, device=x.device) @ torch.randn(256, 256, device=x.device)).sum().item()
    assert graphed.frame_count == eager.frame_count
    assert graphed.build_visible_page_table(0) == eager.build_visible_page_table(0)
    assert graphed.get_cache_stats(0) == eager.get_cache_stats(0)
    for a, b in zip(graphed.kv_caches, eager.kv_caches):
        assert torch.equal(a, b)
    assert graphed.device_header()["error"] == 0
    # and the eager path carries on from the replayed state
    assert torch.equal(f_g(xs[2]), f_e(xs[2]))


def test_graph_refused_outside_the_steady_state():
    from lingbot_map_amd import GraphedFrame
    mk, frame_on, xs, fill = _setup(cross_frame_special=True)
    m = mk()
    f = frame_on(m)
    for i in range(fill + 2):
        f(xs[i % 6])
    # evicted frames leave memory tokens behind: the visible set grows every frame
    assert not m.steady_state(cross_frame_special=True)
    with pytest.raises(RuntimeError):
        GraphedFrame(m, f, [xs[0]], cross_frame_special=True)


def test_device_token_counts_match_host_counts():
    """The same stream through a manager whose kernels read the token counts on the device and
    through the default one: identical tables and pools, outputs within the bf16 bar (the KV
    split may differ), keyframes and read-only frames, trajectory memory growing."""
    from lingbot_map_amd import HipPagedKVCacheManager
    dev = torch.device("cuda:0")
    T, H = 70, 2
    mk = lambda live: HipPagedKVCacheManager(2, 8, T, H, 64, torch.bfloat16, dev, num_special_tokens=5, scale_frames=1,
                                             sliding_window=3, max_total_frames=64, page_size=16, layout="frame_pages",
                                             num_streams=2, device_token_counts=live)
    a, b = mk(False), mk(True)
    g = torch.Generator(device=dev).manual_seed(3)
    for f in range(30):
        keyframe = [f % 4 != 3, f % 5 != 2]
        for blk in range(2):
            q, k, v = (torch.randn(2 * T, H, 64, generator=g, device=dev).to(torch.bfloat16) for _ in range(3))
            ya = a.step(blk, q, k, v, keyframe=keyframe)
            yb = b.step(blk, q, k, v, keyframe=keyframe)
            err = (ya.float() - yb.float()).abs()
            assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3, (f, blk)
    for s in range(2):
        assert a.build_visible_page_table(0, stream=s) == b.build_visible_page_table(0, stream=s)
        assert a.build_visible_page_lens(0, stream=s) == b.build_visible_page_lens(0, stream=s)
    assert a.get_cache_stats(0) == b.get_cache_stats(0)
    for x, y in zip(a.kv_caches, b.kv_caches):
        assert torch.equal(x, y)
    assert a.device_header()["error"] == 0 and b.device_header()["error"] == 0
    assert b.device_header()["plan_kv_tokens"] == a.device_header()["plan_kv_tokens"]


def test_graph_replay_with_growing_trajectory_memory():
    """With device-side token counts a frame whose evictions leave memory tokens behind is
    replayable: eight replays against an eager manager, tables and pools bit for bit, outputs
    within the bf16 bar (the captured launch keeps its KV split while the eager one re-plans)."""
    from lingbot_map_amd import GraphedFrame
    mk, frame_on, xs, fill = _setup(cross_frame_special=True, device_token_counts=True)
    eager, graphed = mk(), mk()
    f_e, f_g = frame_on(eager), frame_on(graphed)
    for i in range(fill + 2):
        f_e(xs[i % 6]); f_g(xs[i % 6])
    assert graphed.steady_state(cross_frame_special=True)
    g = GraphedFrame(graphed, f_g, [xs[0]], cross_frame_special=True)
    tokens0 = eager.device_header()["plan_kv_tokens"]      # the last keyframe's plan
    for i in range(8):
        x = xs[(3 * i + 1) % 6]
        want = f_e(x)
        got = g(x)
        torch.cuda.synchronize()
        # block outputs of magnitude up to several units: two bf16 steps at the top of the range
        err = (got.float() - want.float()).abs()
        assert err.max().item() <= 2 ** -6 * want.float().abs().max().item() and err.mean().item() <= 2e-3, f"replay {i}"
        _ = (torch.randn(256, 256, device=x.device) @ torch.randn(256, 256, device=x.device)).sum().item()
    assert graphed.device_header()["plan_kv_tokens"] == tokens0 + 8 * 5       # five memory tokens per evicted frame
    assert graphed.frame_count == eager.frame_count
    assert graphed.get_cache_stats(0) == eager.get_cache_stats(0)
    assert graphed.build_visible_page_table(0) == eager.build_visible_page_table(0)
    assert graphed.build_visible_page_lens(0) == eager.build_visible_page_lens(0)
    for a, b in zip(graphed.kv_caches, eager.kv_caches):   # K/V of the later blocks inherit those last-bit differences
        assert ((a.float() - b.float()).abs() / b.float().abs().clamp_min(1.0)).max().item() <= 2 ** -5
    assert graphed.device_header()["error"] == 0
    want = f_e(xs[2]).float()
    err = (f_g(xs[2]).float() - want).abs()   # the eager path carries on from the replayed state
    assert err.max().item() <= 2 ** -6 * want.abs().max().item()


def test_keyframe_interval_stream_replayed_as_two_graphs():
    """Keyframe interval 4 in the steady state (K, N, N, N, K, ...): the keyframe graph and the
    read-only graph replayed in that pattern against the eager path - outputs bit for bit, and
    tables, counts and pools identical afterwards; a read-only replay changes no table word."""
    from lingbot_map_amd import GraphedStream, set_skip_append
    mk, frame_on, xs, fill = _setup(cross_frame_special=False)
    eager, graphed = mk(), mk()
    f_e, f_g = frame_on(eager), frame_on(graphed)
    for i in range(fill + 2):
        f_e(xs[i % 6]); f_g(xs[i % 6])
    stream = GraphedStream(graphed, f_g, [xs[0]], cross_frame_special=False)
    assert graphed.frame_count == eager.frame_count and not graphed._skip_append
    for i in range(13):
        keyframe = i % 4 == 0
        x = xs[(5 * i + 2) % 6]
        set_skip_append(eager, not keyframe)
        want = f_e(x)
        tables_before = graphed._tables.clone()
        got = stream(x, keyframe=keyframe)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"frame {i} keyframe={keyframe}"
        if not keyframe:
            assert torch.equal(graphed._tables[..., :11], tables_before[..., :11])
        _ = (torch.randn(128, 128, device=x.device) @ torch.randn(128, 128, device=x.device)).sum().item()
    set_skip_append(eager, False)
    assert graphed.frame_count == eager.frame_count
    assert graphed.build_visible_page_table(0) == eager.build_visible_page_table(0)
    assert graphed.get_cache_stats(0) == eager.get_cache_stats(0)
    for a, b in zip(graphed.kv_caches, eager.kv_caches):
        assert torch.equal(a, b)
    graphed.check_device_errors()
    assert torch.equal(f_g(xs[1]), f_e(xs[1]))      # the eager path carries on from the replayed state


def test_graphed_aggregator_equals_eager_aggregator():
    """The whole aggregator shell (image in, group outputs out) replayed as graphs against the
    same weights run eagerly, two ragged streams, the 3-D rotary table fed per frame."""
    from lingbot_map_amd import GraphedAggregator, HipAggregatorStream, set_skip_append
    dev = torch.device("cuda:0")
    torch.manual_seed(9)
    kw = dict(img_size=56, patch_size=14, embed_dim=128, depth=2, num_heads=2, init_values=0.5, patch_embed="conv",
              enable_3d_rope=True, max_frame_num=64, kv_cache_sliding_window=[2, 3], kv_cache_scale_frames=1,
              kv_cache_cross_frame_special=False, use_scale_token=False, page_size=4, layout="frame_pages", num_streams=2)
    a = HipAggregatorStream(**kw).to(dev, torch.bfloat16).eval()
    b = HipAggregatorStream(**kw).to(dev, torch.bfloat16).eval()
    b.load_state_dict(a.state_dict())
    g = torch.Generator(device=dev).manual_seed(10)
    imgs = [torch.rand(2, 1, 3, 42, 56, generator=g, device=dev).to(torch.bfloat16) for _ in range(5)]
    with torch.no_grad():
        for i in range(6):                       # anchor and both windows full
            a(imgs[i % 5]); b(imgs[i % 5])
        graphed = GraphedAggregator(b, imgs[0], selected_idx=[1])
        assert b.total_frames_processed == a.total_frames_processed == 6
        for i in range(9):
            keyframe = i % 3 != 1
            set_skip_append(a.kv_cache_manager, not keyframe)
            want = a(imgs[(2 * i + 1) % 5], selected_idx=[1])[0][0]
            got = graphed(imgs[(2 * i + 1) % 5], keyframe=keyframe)[0]
            torch.cuda.synchronize()
            assert torch.equal(got, want), (i, keyframe)
    assert a.total_frames_processed == b.total_frames_processed == 12
    ma, mb = a.kv_cache_manager, b.kv_cache_manager
    for s in range(2):
        assert ma.build_visible_page_table(0, stream=s) == mb.build_visible_page_table(0, stream=s)
    for x, y in zip(ma.kv_caches, mb.kv_caches):
        assert torch.equal(x, y)
    mb.check_device_errors()


def test_pipelined_aggregator_equals_eager_aggregator():
    """The next frame's image encoder as a second branch of the graph that takes the present frame
    through its frame and global blocks: the outputs are those of the eager aggregator bit for
    bit, one call later; keyframes and read-only frames mixed, two ragged streams, an encoder
    with blocks of its own (whose fc2 splits K, so both branches use a K-split workspace)."""
    from lingbot_map_amd import HipAggregatorStream, PipelinedAggregator, set_skip_append
    dev = torch.device("cuda:0")
    torch.manual_seed(11)
    kw = dict(img_size=56, patch_size=14, embed_dim=128, depth=2, num_heads=2, init_values=0.5, patch_embed="vit",
              encoder_depth=2, enable_3d_rope=True, max_frame_num=64, kv_cache_sliding_window=[2, 3], kv_cache_scale_frames=1,
              kv_cache_cross_frame_special=False, use_scale_token=False, page_size=4, layout="frame_pages", num_streams=2)
    a = HipAggregatorStream(**kw).to(dev, torch.bfloat16).eval()
    b = HipAggregatorStream(**kw).to(dev, torch.bfloat16).eval()
    b.load_state_dict(a.state_dict())
    g = torch.Generator(device=dev).manual_seed(12)
    imgs = [torch.rand(2, 1, 3, 42, 56, generator=g, device=dev).to(torch.bfloat16) for _ in range(5)]
    with torch.no_grad():
        for i in range(6):                       # anchor and both windows full
            a(imgs[i % 5]); b(imgs[i % 5])
        piped = PipelinedAggregator(b, imgs[0], selected_idx=[1])
        with pytest.raises(RuntimeError):
            piped(imgs[0])
        frames = [imgs[(2 * i + 1) % 5] for i in range(10)]
        piped.prime(frames[0])
        for i in range(9):
            keyframe = i % 3 != 1
            set_skip_append(a.kv_cache_manager, not keyframe)
            want = a(frames[i], selected_idx=[1])[0][0]
            got = piped(frames[i + 1], keyframe=keyframe)[0]       # frame i comes out while frame i + 1 is encoded
            torch.cuda.synchronize()
            assert torch.equal(got, want), (i, keyframe)
    assert a.total_frames_processed == b.total_frames_processed == 12
    for x, y in zip(a.kv_cache_manager.kv_caches, b.kv_cache_manager.kv_caches):
        assert torch.equal(x, y)
    b.kv_cache_manager.check_device_errors()
