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
    g = GraphedFrame(graphed, f_g, [xs[0]], cross_frame_special=False)   # runs one eager frame with xs[0] itself
    f_e(xs[0])
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
    f_e(xs[0])
    tokens0 = graphed.device_header()["plan_kv_tokens"]
    for i in range(8):
        x = xs[(3 * i + 1) % 6]
        want = f_e(x)
        got = g(x)
        torch.cuda.synchronize()
        err = (got.float() - want.float()).abs()
        assert err.max().item() <= 3e-2 and err.mean().item() <= 2e-3, f"replay {i}"
        _ = (torch.randn(256, 256, device=x.device) @ torch.randn(256, 256, device=x.device)).sum().item()
    assert graphed.device_header()["plan_kv_tokens"] == tokens0 + 8 * 5       # five memory tokens per evicted frame
    assert graphed.frame_count == eager.frame_count
    assert graphed.get_cache_stats(0) == eager.get_cache_stats(0)
    assert graphed.build_visible_page_table(0) == eager.build_visible_page_table(0)
    assert graphed.build_visible_page_lens(0) == eager.build_visible_page_lens(0)
    for a, b in zip(graphed.kv_caches, eager.kv_caches):
        assert ((a.float() - b.float()).abs() / b.float().abs().clamp_min(1.0)).max().item() <= 2 ** -6
    assert graphed.device_header()["error"] == 0
    err = (f_g(xs[2]).float() - f_e(xs[2]).float()).abs()   # the eager path carries on from the replayed state
    assert err.max().item() <= 3e-2
