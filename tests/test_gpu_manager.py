"""The drop-in manager on the GPU against the oracle: device page tables bit-exact after
every operation, pool contents exact, attention within the bf16 tolerance."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

BF16_MAX_ABS, BF16_MEAN_ABS = 2e-2, 2e-3


def make(layout, page_size, T=7, n_sp=3, scale=1, window=2, max_total=6, H=2, blocks=2, **kw):
    from lingbot_map_amd import HipPagedKVCacheManager
    return HipPagedKVCacheManager(blocks, scale + window + 16, T, H, 64, torch.bfloat16, torch.device("cuda:0"),
                                  num_special_tokens=n_sp, scale_frames=scale, sliding_window=window,
                                  max_total_frames=max_total, page_size=page_size, layout=layout, **kw)


def frame(T, H, g):
    return tuple(torch.randn(T, H, 64, generator=g).to(torch.bfloat16) for _ in range(3))


def test_six_frame_trace_on_device():
    """Hand-derived ids for tokens_per_frame 7 (see tests/test_oracle_policy.py)."""
    m = make("two_stream", None)
    assert m.page_size == 4 and m.max_patch_pages == 19 and m.max_num_pages == 40
    g = torch.Generator().manual_seed(0)
    visible = [[18, 39], [18, 17, 39, 38], [18, 17, 16, 39, 38, 37], [18, 16, 15, 39, 38, 37],
               [18, 15, 17, 39, 38, 37, 36], [18, 17, 16, 39, 38, 37, 36, 35]]
    last = [3, 2, 1, 4, 3, 2]
    for vis, ll in zip(visible, last):
        q, k, v = frame(7, 2, g)
        m.append_frame(0, k.cuda(), v.cuda())
        m.evict_frames(0, 1, 2)
        assert m.build_visible_page_table(0) == vis
        assert m.compute_last_page_len(0) == ll
        assert m.device_header()["error"] == 0
    assert m.get_cache_stats() == {"frame_count": 6, "scale_pages": 1, "live_pages": 2, "free_pages": 16,
                                   "special_tokens": 18}
    # non-keyframe probe: append, look, roll back -> bit-identical tables
    before = m._tables.clone()
    m._defer_eviction = True
    q, k, v = frame(7, 2, g)
    m.append_frame(0, k.cuda(), v.cuda())
    m.evict_frames(0, 1, 2)
    assert m.build_visible_page_table(0) == [18, 17, 16, 15, 39, 38, 37, 36, 35, 34]
    assert m.compute_last_page_len(0) == 1
    m.rollback_last_frame(0)
    m._defer_eviction = False
    hdr_plan = slice(11, 13)
    a, b = m._tables.clone(), before
    a[..., hdr_plan] = 0; b[..., hdr_plan] = 0
    n_free = m.device_header()["n_free_patch"]
    assert torch.equal(a[0, 0, :16 + n_free], b[0, 0, :16 + n_free])
    assert m.build_visible_page_table(0) == visible[-1]
    m.reset()
    assert m.frame_count == [0, 0] and m.device_header()["frame_count"] == 0


def test_reference_sanity_check_figures_on_device():
    # lingbot_map/layers/flashinfer_cache.py:577-656, run the reference's way: block by block
    m = make("two_stream", None, T=262, n_sp=6, scale=8, window=64, max_total=200, H=16, per_block_tables=True)
    g = torch.Generator().manual_seed(0)
    for block in range(2):
        for t in range(100):
            _, k, v = frame(262, 16, g)
            m.append_frame(block, k.cuda(), v.cuda())
            m.evict_frames(block, scale_frames=8, sliding_window=64)
        st = m.get_cache_stats(block)
        assert st["scale_pages"] == 8 and st["live_pages"] == 64 and st["special_tokens"] == 600
        vis = m.build_visible_page_table(block)
        assert len(vis) == 8 + 64 + 3
        assert all(p < m.max_patch_pages for p in vis[:72]) and all(p >= m.max_patch_pages for p in vis[72:])
        assert m.compute_last_page_len(block) == 88
        assert m.device_header(block)["error"] == 0
    q0, q1 = frame(262, 16, g)[0].cuda(), frame(262, 16, g)[0].cuda()
    assert m.compute_attention(0, q0).shape == (262, 16, 64)
    assert m.compute_attention(1, q1).shape == (262, 16, 64)
    m.reset()
    assert m.frame_count[0] == 0


def test_error_conventions():
    m = make("two_stream", None)
    q = torch.zeros(7, 2, 64, dtype=torch.bfloat16, device="cuda")
    assert torch.equal(m.compute_attention(0, q), torch.zeros_like(q))   # nothing cached -> zeros
    with pytest.raises(AssertionError, match="cannot rollback"):
        m.rollback_last_frame(0)
    m._defer_eviction = True
    for _ in range(19):
        m.append_frame(0, q, q)
    with pytest.raises(AssertionError, match="patch page pool exhausted"):
        m.append_frame(0, q, q)
    assert m.device_header()["error"] == 0     # the host refused before the device saw it
    with pytest.raises(AssertionError):
        m.append_frame(0, q[:5], q[:5])


def test_device_error_word_is_raised_by_the_product_path():
    """The device tables keep a sticky error word; the manager raises it as the reference's
    AssertionError wherever it already waits for the device (table read-back, reset) and on
    request.  Here the host's count mirror is made to disagree with the device on purpose -
    one special token too many - so the plan step records LBM_TERR_KV_COUNT; the kernels only
    ever read as many rows as the table holds."""
    m = make("two_stream", None)
    q = torch.zeros(7, 2, 64, dtype=torch.bfloat16, device="cuda")
    m.append_frame(0, q, q)
    m.check_device_errors()                      # clean so far
    m._counts[0][0].special_tokens += 1          # the host now expects one visible token too many
    m.compute_attention(0, q)                    # plans with the wrong expectation
    with pytest.raises(AssertionError, match="visible token count mismatch"):
        m.check_device_errors()
    with pytest.raises(AssertionError, match="visible token count mismatch"):
        m.build_visible_page_table(0)
    with pytest.raises(AssertionError, match="visible token count mismatch"):
        m.reset()                                # resets, then reports what the old sequence recorded
    assert m.frame_count[0] == 0 and m.device_header()["error"] == 0
    m.append_frame(0, q, q)
    m.reset()                                    # nothing recorded: no raise


def test_table_read_back_leaves_the_live_plan_alone():
    """build_visible_page_table & co. between the blocks of a non-keyframe: the row table and
    the device-side token count the later blocks attend through are those of the frame's plan
    (cache plus the frame's own rows), not the read-back's."""
    T, n_sp, H = 21, 5, 2
    m = make("frame_pages", 4, T=T, n_sp=n_sp, scale=1, window=2, max_total=32, H=H, blocks=2, device_token_counts=True)
    g = torch.Generator().manual_seed(4)
    for _ in range(3):
        for b in range(2):
            q, k, v = frame(T, H, g)
            m.step(b, q.cuda(), k.cuda(), v.cuda(), keyframe=[True])
    q, k, v = (x.cuda() for x in frame(T, H, g))
    m.step(0, q, k, v, keyframe=[False])
    rows_before = m._kv_rows[0].clone()
    count_before = m.device_header()["plan_kv_tokens"]
    assert count_before == 3 * T + T             # three cached frames and the frame's own rows
    ids = m.build_visible_page_table(0)
    assert len(ids) == 3 * math.ceil(T / 4)
    assert m.compute_last_page_len(0) == T - (math.ceil(T / 4) - 1) * 4
    assert torch.equal(m._kv_rows[0], rows_before)
    assert m.device_header()["plan_kv_tokens"] == count_before
    out1 = m.step(1, q, k, v, keyframe=[False])
    assert torch.isfinite(out1.float()).all()


@pytest.mark.parametrize("layout,page_size", [("two_stream", None), ("two_stream", 16), ("frame_pages", 16)])
@pytest.mark.parametrize("interval,native_tail", [(1, False), (3, False), (3, True)])
def test_stream_against_oracle(layout, page_size, interval, native_tail):
    """40 frames, 3 blocks sharing one table set: ids, pool and outputs against the oracle."""
    from oracle.page_policy import PagePolicy, is_keyframe
    from oracle.sdpa_cache import PagedStreamOracle
    T, n_sp, scale, window, H, blocks = 53, 5, 2, 3, 4, 3
    m = make(layout, page_size, T=T, n_sp=n_sp, scale=scale, window=window, max_total=64, H=H, blocks=blocks)
    pol = [PagePolicy(T, n_sp, page_size, scale, window, 64, layout=layout) for _ in range(blocks)]
    orc = [PagedStreamOracle(p, H, 64, torch.bfloat16) for p in pol]
    g = torch.Generator().manual_seed(11)
    for f in range(40):
        kf = is_keyframe(f, scale, interval)
        for b in range(blocks):
            q, k, v = frame(T, H, g)
            ref = orc[b].step(q, k, v, keyframe=kf)
            qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
            if kf:
                m.append_frame(b, kd, vd)
                m.evict_frames(b, scale, window)
                out = m.compute_attention(b, qd)
            elif native_tail:
                out = m.compute_attention(b, qd, kd, vd)
            else:   # the reference block's non-keyframe sequence (block.py:257-263)
                prev = m._defer_eviction
                m._defer_eviction = True
                m.append_frame(b, kd, vd)
                out = m.compute_attention(b, qd)
                m.rollback_last_frame(b)
                m._defer_eviction = prev
            err = (out.float().cpu() - ref.float()).abs()
            assert err.max().item() <= BF16_MAX_ABS and err.mean().item() <= BF16_MEAN_ABS, (f, b, err.max().item())
        assert m.build_visible_page_table(0) == pol[0].build_visible_page_table(), f"frame {f}"
        assert m.build_visible_page_lens(0) == pol[0].build_visible_page_lens()
        assert m.device_header()["error"] == 0
        st = m.get_cache_stats(0)
        assert st == pol[0].get_cache_stats()
    # every live page holds exactly what the oracle's pool holds
    for b in range(blocks):
        ids, lens = pol[b].build_visible_page_table(), pol[b].build_visible_page_lens()
        dev_pool = m.kv_caches[b].cpu()
        for p, n in zip(ids, lens):
            assert torch.equal(dev_pool[p, :, :n], orc[b].pool[p, :, :n])


def test_fused_step_matches_method_by_method():
    from oracle.page_policy import is_keyframe
    T, n_sp, scale, window, H = 53, 5, 1, 4, 4
    a = make("frame_pages", 16, T=T, n_sp=n_sp, scale=scale, window=window, max_total=64, H=H, blocks=2)
    b = make("frame_pages", 16, T=T, n_sp=n_sp, scale=scale, window=window, max_total=64, H=H, blocks=2)
    g = torch.Generator().manual_seed(21)
    for f in range(30):
        kf = is_keyframe(f, scale, 4)
        for blk in range(2):
            q, k, v = (x.cuda() for x in frame(T, H, g))
            if kf:
                a.append_frame(blk, k, v); a.evict_frames(blk, scale, window); ref = a.compute_attention(blk, q)
            else:
                ref = a.compute_attention(blk, q, k, v)
            out = b.step(blk, q, k, v, keyframe=[kf])
            assert torch.equal(out, ref)
        assert torch.equal(a._tables[..., :11], b._tables[..., :11])
        assert a.build_visible_page_table(0) == b.build_visible_page_table(0)
    assert torch.equal(a.kv_caches[1], b.kv_caches[1])


@pytest.mark.parametrize("layout,page_size", [("two_stream", None), ("frame_pages", 16)])
def test_flow_keyframe_protocol_of_the_windowed_driver(layout, page_size):
    """The windowed driver decides after the forward pass whether a frame is a keyframe
    (lingbot_map/models/gct_stream_window.py:362-420): eviction is deferred, every block appends
    and attends, then either every block rolls the frame back or every block runs the deferred
    eviction; the cache is reset between windows.  Ids, counters, pool and outputs against the
    oracle after every frame."""
    from oracle.page_policy import PagePolicy
    from oracle.sdpa_cache import PagedStreamOracle
    T, n_sp, scale, window, H, blocks = 53, 5, 2, 3, 4, 3
    m = make(layout, page_size, T=T, n_sp=n_sp, scale=scale, window=window, max_total=64, H=H, blocks=blocks)
    pol = [PagePolicy(T, n_sp, page_size, scale, window, 64, layout=layout) for _ in range(blocks)]
    orc = [PagedStreamOracle(p, H, 64, torch.bfloat16) for p in pol]
    g = torch.Generator().manual_seed(19)
    for win in range(2):
        for f in range(18):
            accept = f < scale or bool(torch.rand(1, generator=g).item() < 0.6)
            m._defer_eviction = True
            for p in pol:
                p._defer_eviction = True
            for b in range(blocks):
                q, k, v = frame(T, H, g)
                orc[b].append_frame(k, v)
                pol[b].evict_frames(scale, window)               # suppressed while deferred
                ref = orc[b].compute_attention(q)
                m.append_frame(b, k.cuda(), v.cuda())
                m.evict_frames(b, scale, window)
                out = m.compute_attention(b, q.cuda())
                err = (out.float().cpu() - ref.float()).abs()
                assert err.max().item() <= BF16_MAX_ABS and err.mean().item() <= BF16_MEAN_ABS, (win, f, b)
            for b in range(blocks):
                if accept:
                    m.execute_deferred_eviction(b, scale_frames=scale, sliding_window=window)
                    pol[b].execute_deferred_eviction(scale, window)
                else:
                    m.rollback_last_frame(b)
                    pol[b].rollback_last_frame()
            m._defer_eviction = False
            for p in pol:
                p._defer_eviction = False
            assert m.build_visible_page_table(0) == pol[0].build_visible_page_table(), (win, f)
            assert m.build_visible_page_lens(0) == pol[0].build_visible_page_lens()
            assert m.get_cache_stats(0) == pol[0].get_cache_stats()
            assert m.device_header()["error"] == 0
        for b in range(blocks):
            ids, lens = pol[b].build_visible_page_table(), pol[b].build_visible_page_lens()
            dev_pool = m.kv_caches[b].cpu()
            for p, n in zip(ids, lens):
                assert torch.equal(dev_pool[p, :, :n], orc[b].pool[p, :, :n])
        m.reset()
        for p in pol:
            p.reset()
        assert m.num_frames == 0 and m.build_visible_page_table(0) == []


@pytest.mark.parametrize("T,H,streams,dtype", [(1004, 16, 1, torch.bfloat16), (203, 4, 3, torch.bfloat16),
                                               (70, 2, 2, torch.float32), (7, 2, 1, torch.bfloat16)])
def test_step_that_appends_inside_the_attention_call(T, H, streams, dtype):
    """step() with the append carried by the attention call (the row table names the new frame by
    the caller's rows, lbm_attn_run_append stores them once the pool was read) against step() with
    the append as a launch of its own in front (fuse_append = False): the same outputs bit for bit,
    the same pools, the same tables - anchor, sliding windows of different lengths, evictions that
    hand pages out again, keyframes and read-only frames mixed per stream, an inactive stream,
    three blocks behind one table; split-KV with the combine launch (1,004 tokens), the short-KV
    kernel and the fp32 kernels (append behind the attention), and one stream of 7 tokens."""
    from lingbot_map_amd import HipPagedKVCacheManager
    dev = torch.device("cuda:0")
    kw = dict(num_special_tokens=3, scale_frames=1, sliding_window=[4, 2, 3][:streams] if streams > 1 else 4,
              max_total_frames=64, page_size=16, layout="frame_pages", num_streams=streams, force_fp32=dtype == torch.float32)
    a = HipPagedKVCacheManager(3, 24, T, H, 64, dtype, dev, **kw)
    b = HipPagedKVCacheManager(3, 24, T, H, 64, dtype, dev, **kw)
    b.fuse_append = False
    g = torch.Generator(device=dev).manual_seed(T + H)
    for i in range(9):
        keyframe = [(i + s) % 4 != 2 or i < 2 for s in range(streams)]
        if streams == 3 and i == 5:
            a.set_active_streams([True, False, True]); b.set_active_streams([True, False, True])
        if streams == 3 and i == 6:
            a.set_active_streams(None); b.set_active_streams(None)
        for blk in range(3):
            q, k, v = (torch.randn(streams * T, H, 64, generator=g, device=dev).to(dtype) / (2 if j else 1) for j in range(3))
            oa = a.step(blk, q, k, v, keyframe=keyframe, cross_frame_special=False)
            ob = b.step(blk, q, k, v, keyframe=keyframe, cross_frame_special=False)
            torch.cuda.synchronize()
            assert torch.isfinite(oa.float()).all() and torch.equal(oa, ob), (i, blk)
        assert a._newest_self[0] == any(keyframe) and not b._newest_self[0]
    for x, y in zip(a.kv_caches, b.kv_caches):
        assert torch.equal(x, y)
    assert torch.equal(a._tables, b._tables)
    for s in range(streams):
        assert a.build_visible_page_table(0, stream=s) == b.build_visible_page_table(0, stream=s)
    a.check_device_errors(); b.check_device_errors()
    # a block that does not go through step() on a frame that step() led is refused
    q, k, v = (torch.randn(streams * T, H, 64, generator=g, device=dev).to(dtype) for _ in range(3))
    a.step(0, q, k, v, keyframe=[True] * streams, cross_frame_special=False)
    with pytest.raises(RuntimeError):
        a._attend_planned(1, q, None, None)
