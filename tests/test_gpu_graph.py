"""A steady-state streamed frame captured as a HIP graph replays to the same results as the
eager path: outputs bit for bit on every replay (with eager work and synchronisations in
between), device page tables and pools identical afterwards."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _setup(cross_frame_special):
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
                                        layout="frame_pages")
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
