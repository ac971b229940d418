"""The benchmark configurations as parity cases (GPU), each against the CPU oracle.

config 1  fp32, 8 streamed frames of 1004 tokens, 16 heads: max-abs <= 1e-5 vs fp32 SDPA
config 3  trajectory memory over non-contiguous pages, page-table order shuffled (reduced
          frame count; the full 10,000-frame table is checked index-only)
config 4  keyframe interval 4 over 320 frames: page ids bit-exact after every step
config 5  four streams with windows 4/8/16/16 batched in one launch
"""
import ctypes as C
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

BF16_MAX_ABS, BF16_MEAN_ABS = 2e-2, 2e-3
FP32_MAX_ABS = 1e-5


def manager(**kw):
    from lingbot_map_amd import HipPagedKVCacheManager
    args = dict(num_blocks=1, max_num_frames=33, tokens_per_frame=1004, num_heads=16, head_dim=64,
                dtype=torch.bfloat16, device=torch.device("cuda:0"), num_special_tokens=5, scale_frames=1,
                sliding_window=16, max_total_frames=64, page_size=16, layout="frame_pages")
    args.update(kw)
    return HipPagedKVCacheManager(**args)


def test_config1_fp32_eight_frames():
    from oracle.sdpa_cache import sdpa_nhd
    m = manager(dtype=torch.float32, force_fp32=True)
    assert m.dtype == torch.float32
    torch.manual_seed(0)
    ks, vs = [], []
    for f in range(8):
        q, k, v = (torch.randn(1004, 16, 64) / 8 for _ in range(3))
        ks.append(k); vs.append(v)
        m.append_frame(0, k.cuda(), v.cuda())
        m.evict_frames(0, 1, 16)
        out = m.compute_attention(0, q.cuda())
        ref = sdpa_nhd(q, torch.cat(ks), torch.cat(vs))
        err = (out.cpu() - ref).abs().max().item()
        assert out.dtype == torch.float32 and err <= FP32_MAX_ABS, (f, err)
    assert m.device_header()["error"] == 0


def test_fp32_ragged_pages_against_float64_loops():
    from lingbot_map_amd import _native as N
    from oracle.sdpa_cache import gather_paged, naive_attention_f64
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(4)
    S, H, D, tq = 4, 2, 64, 9
    pool = torch.randn(7, 2, S, H, D, generator=g)
    q = torch.randn(tq, H, D, generator=g)
    ids, lens = [5, 0, 3, 6], [4, 1, 3, 2]
    kk, vv = gather_paged(pool, ids, lens)
    ref = torch.from_numpy(naive_attention_f64(q.numpy(), kk.numpy(), vv.numpy())).float()
    rows = torch.tensor([p * 2 * S + s for p, n in zip(ids, lens) for s in range(n)], dtype=torch.int32, device=dev)
    qd, pd = q.to(dev), pool.to(dev)
    out = torch.empty_like(qd)
    st = (N.AttnStream * 1)(N.AttnStream(0, tq, 0, rows.numel()))
    ws = torch.empty(1024, dtype=torch.uint8, device=dev)
    p = lambda t: C.c_void_p(t.data_ptr())
    N.check(N.lib.lbm_attn_run(p(qd), p(pd), p(out), None, None, p(rows), st, 1, H, D, S, N.DTYPE_F32,
                               1 / math.sqrt(D), p(ws), ws.numel(), None))
    torch.cuda.synchronize()
    assert (out.cpu() - ref).abs().max().item() <= FP32_MAX_ABS


def test_config3_memory_pages_shuffled_table():
    """Frames leaving the window keep 5 tokens in place; the visible table (anchor, window,
    memory pages with 5 valid slots each) is then permuted and must give the same output."""
    from lingbot_map_amd import _native as N
    from oracle.page_policy import PagePolicy
    from oracle.sdpa_cache import PagedStreamOracle
    T, H, window, frames = 1004, 16, 16, 40
    m = manager(max_total_frames=64)
    pol = PagePolicy(T, 5, 16, 1, window, 64, layout="frame_pages")
    orc = PagedStreamOracle(pol, H, 64, torch.bfloat16)
    g = torch.Generator().manual_seed(2)
    for f in range(frames):
        q, k, v = (torch.randn(T, H, 64, generator=g).to(torch.bfloat16) for _ in range(3))
        if f < frames - 1:      # only the last step is compared numerically (CPU oracle time)
            plan = pol.append_frame(); pol.evict_frames(1, window)
            from oracle.sdpa_cache import write_frame
            write_frame(orc.pool, plan.page, plan.slot, k, v)
            m.append_frame(0, k.cuda(), v.cuda()); m.evict_frames(0, 1, window)
            continue
        ref = orc.step(q, k, v)
        out = m.step(0, q.cuda(), k.cuda(), v.cuda())
    ids, lens = m.build_visible_page_table(0), m.build_visible_page_lens(0)
    assert ids == pol.build_visible_page_table() and lens == pol.build_visible_page_lens()
    n_mem = frames - 1 - window
    assert lens[-n_mem:] == [5] * n_mem and sum(lens) == 17 * T + 5 * n_mem
    err = (out.float().cpu() - ref.float()).abs()
    assert err.max().item() <= BF16_MAX_ABS and err.mean().item() <= BF16_MEAN_ABS
    # shuffled page-table order through the general entry points
    perm = torch.randperm(len(ids), generator=g).tolist()
    dev = torch.device("cuda:0")
    ids_d = torch.tensor([ids[i] for i in perm], dtype=torch.int32, device=dev)
    lens_d = torch.tensor([lens[i] for i in perm], dtype=torch.int32, device=dev)
    n_tok = sum(lens)
    rows = torch.empty(n_tok, dtype=torch.int32, device=dev)
    i32 = C.c_int32
    p = lambda t: C.c_void_p(t.data_ptr())
    N.check(N.lib.lbm_rows_from_pages(p(ids_d), p(lens_d), (i32 * 2)(0, len(ids)), (i32 * 1)(n_tok), (i32 * 1)(0),
                                      1, 16, p(rows), None))
    qd = q.cuda()
    out2 = torch.empty_like(qd)
    st = (N.AttnStream * 1)(N.AttnStream(0, T, 0, n_tok))
    need = N.lib.lbm_attn_workspace_bytes(st, 1, H, 64)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    N.check(N.lib.lbm_attn_run(p(qd), p(m.kv_caches[0]), p(out2), None, None, p(rows), st, 1, H, 64, 16,
                               N.DTYPE_BF16, 0.125, p(ws), ws.numel(), None))
    torch.cuda.synchronize()
    err2 = (out2.float().cpu() - ref.float()).abs()
    assert err2.max().item() <= BF16_MAX_ABS and err2.mean().item() <= BF16_MEAN_ABS


def test_config3_ten_thousand_frame_tables():
    """The 10,000-frame stream, index-only: device tables against the oracle at checkpoints."""
    from oracle.page_policy import PagePolicy
    T, H = 37, 1     # small frames keep the pool small; the table logic does not depend on T
    m = manager(tokens_per_frame=T, num_heads=H, max_total_frames=10000, sliding_window=16)
    pol = PagePolicy(T, 5, 16, 1, 16, 10000, layout="frame_pages")
    k = torch.zeros(T, H, 64, dtype=torch.bfloat16, device="cuda")
    for f in range(10000):
        pol.append_frame(); pol.evict_frames(1, 16)
        m.append_frame(0, k, k); m.evict_frames(0, 1, 16)
        if f in (0, 16, 17, 18, 999, 5000, 9999):
            assert m.build_visible_page_table(0) == pol.build_visible_page_table(), f
            assert m.build_visible_page_lens(0) == pol.build_visible_page_lens(), f
    st = m.get_cache_stats()
    assert st["special_tokens"] == 5 * (10000 - 17) and st == pol.get_cache_stats()
    assert m.device_header()["error"] == 0 and m.device_header()["n_memory"] == 10000 - 17


def test_config4_keyframe_interval_indices():
    """320 frames, keyframe interval 4: 1 anchor + 80 keyframes are cached, non-keyframes attend
    read-only; tables bit-exact after every step, outputs checked on a reduced frame size."""
    from oracle.page_policy import PagePolicy, is_keyframe
    from oracle.sdpa_cache import PagedStreamOracle
    T, H = 69, 2
    m = manager(tokens_per_frame=T, num_heads=H, max_total_frames=128)
    pol = PagePolicy(T, 5, 16, 1, 16, 128, layout="frame_pages")
    orc = PagedStreamOracle(pol, H, 64, torch.bfloat16)
    g = torch.Generator().manual_seed(3)
    appended = 0
    for f in range(320):
        kf = is_keyframe(f, 1, 4)
        appended += kf
        q, k, v = (torch.randn(T, H, 64, generator=g).to(torch.bfloat16) for _ in range(3))
        ref = orc.step(q, k, v, keyframe=kf)
        before = m._tables.clone() if not kf else None
        out = m.step(0, q.cuda(), k.cuda(), v.cuda(), keyframe=[kf])
        if not kf:   # a non-keyframe leaves every table word and every pool byte alone
            assert torch.equal(m._tables[..., :11], before[..., :11])
        err = (out.float().cpu() - ref.float()).abs()
        assert err.max().item() <= BF16_MAX_ABS and err.mean().item() <= BF16_MEAN_ABS, f
        if f % 16 == 0 or f > 300:
            assert m.build_visible_page_table(0) == pol.build_visible_page_table(), f
            assert m.build_visible_page_lens(0) == pol.build_visible_page_lens(), f
    assert appended == 81 and m.frame_count[0] == 81 and m.get_cache_stats() == pol.get_cache_stats()
    assert m.device_header()["error"] == 0


def test_config5_four_ragged_streams():
    """Windows 4/8/16/16 (+1 anchor): one launch per kernel for all four streams."""
    from oracle.page_policy import PagePolicy
    from oracle.sdpa_cache import PagedStreamOracle
    T, H, windows = 1004, 16, [4, 8, 16, 16]
    m = manager(num_streams=4, sliding_window=windows, max_total_frames=32)
    # every stream's pool is sized for the largest window; the stream's own window only
    # decides when frames leave it
    pols = [PagePolicy(T, 5, 16, 1, 16, 32, layout="frame_pages", page_base=b * m.max_num_pages) for b in range(4)]
    assert all(p.max_num_pages == m.max_num_pages for p in pols)
    orcs = [PagedStreamOracle(p, H, 64, torch.bfloat16) for p in pols]
    g = torch.Generator().manual_seed(4)
    for f in range(19):
        q, k, v = (torch.randn(4 * T, H, 64, generator=g).to(torch.bfloat16) for _ in range(3))
        out = m.step(0, q.cuda(), k.cuda(), v.cuda())
        for b in range(4):
            sl = slice(b * T, (b + 1) * T)
            orcs[b].append_frame(k[sl], v[sl])
            pols[b].evict_frames(1, windows[b])
            if f == 18:
                ref = orcs[b].compute_attention(q[sl])
                err = (out[sl].float().cpu() - ref.float()).abs()
                assert err.max().item() <= BF16_MAX_ABS and err.mean().item() <= BF16_MEAN_ABS, b
    for b in range(4):
        assert m.build_visible_page_table(0, stream=b) == pols[b].build_visible_page_table()
        assert m.build_visible_page_lens(0, stream=b) == pols[b].build_visible_page_lens()
        assert pols[b].visible_tokens() == (1 + windows[b]) * T + 5 * (19 - 1 - windows[b])
    assert m.device_header()["error"] == 0


@pytest.mark.parametrize("layout,page_size", [("two_stream", None), ("frame_pages", 1), ("frame_pages", 8)])
def test_camera_head_cache_one_token_per_frame_head_dim_128(layout, page_size):
    """The camera head keeps one token per frame in 16 heads of 128 and never evicts
    (lingbot_map/heads/camera_head.py:284-377; lingbot_map/layers/attention.py:307: its eviction
    guard is false for one-token frames), in fp32.  The same manager holds that cache: every
    frame appends one token per block and attends to all of them; 1e-5 against float64."""
    from lingbot_map_amd import HipPagedKVCacheManager
    dev = torch.device("cuda:0")
    H, D, blocks, frames = 16, 128, 4, 150
    m = HipPagedKVCacheManager(blocks, frames + 8, 1, H, D, torch.float32, dev, num_special_tokens=0, scale_frames=8,
                               sliding_window=frames, max_total_frames=frames + 8, force_fp32=True,
                               page_size=page_size, layout=layout)
    assert m.dtype == torch.float32
    g = torch.Generator().manual_seed(21)
    ks = [[] for _ in range(blocks)]
    vs = [[] for _ in range(blocks)]
    for f in range(frames):
        for b in range(blocks):
            q, k, v = (torch.randn(1, H, D, generator=g) for _ in range(3))
            ks[b].append(k); vs[b].append(v)
            m.append_frame(b, k.to(dev), v.to(dev))
            m.evict_frames(b, 8, frames)
            out = m.compute_attention(b, q.to(dev)).cpu()
            if f % 37 == 0 or f == frames - 1:
                K, V = torch.cat(ks[b]).double(), torch.cat(vs[b]).double()          # [f+1, H, D]
                s = torch.einsum("qhd,khd->hqk", q.double(), K) / D ** 0.5
                ref = torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), V)
                assert (out.double() - ref).abs().max().item() <= 1e-5, (f, b)
    assert m.num_frames == frames and m.device_header()["error"] == 0
