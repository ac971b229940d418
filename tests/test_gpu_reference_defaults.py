"""The drop-in at the reference's own defaults, at full size (GPU).

Every other full-size test uses the shapes of the benchmark configurations (1004 tokens per
frame, 16-token pages, whole frames in pages).  Here the manager is built the way
``AggregatorStream._get_kv_cache_manager`` builds the reference's
(lingbot_map/aggregator/stream.py:198-234, lingbot_map/layers/flashinfer_cache.py:100-106):
``two_stream`` layout, ``page_size = patches per frame`` = 999, 6 special tokens (1005 tokens per
frame at 518 x 378), 8 anchor frames and a window of 64, so a steady-state frame attends to
72 x 999 patch tokens plus the packed special stream: about 72,500 KV tokens in 999-token
pages.  Page ids must be the reference allocator's sequence bit for bit; attention is compared
with the oracle's gather + SDPA.

Also here: the multi-frame anchor pass (attention.py:475-511) at the reference's default of 8
frames per stream, which runs on the producer and the paged kernel over the streams' own rows.

Tolerances as in test_gpu_full_size.py: ids, lengths and counts bit-exact; bf16 outputs max-abs
<= 2e-2, mean-abs <= 2e-3 and <= 1 % of the reference's mean magnitude."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

BF16_MAX_ABS, BF16_MEAN_ABS, REL_MEAN = 2e-2, 2e-3, 0.01
T, H, D, N_SP, ANCHOR, WINDOW, MAX_TOTAL = 1005, 16, 64, 6, 8, 64, 200


def check(out, ref, what):
    err = (out.float().cpu() - ref.float()).abs()
    assert torch.isfinite(out.float()).all(), what
    assert err.max().item() <= BF16_MAX_ABS, (what, err.max().item())
    assert err.mean().item() <= BF16_MEAN_ABS, (what, err.mean().item())
    assert err.mean().item() <= REL_MEAN * ref.float().abs().mean().item(), (what, err.mean().item(), ref.float().abs().mean().item())


class ReferenceSurfaceOnly:
    """The manager behind the reference's call surface alone (no ``step`` / ``step_qkv``), so that
    ``HipPagedAttention.stream_attend`` takes the reference's method-by-method sequence
    (lingbot_map/layers/block.py:256-278)."""
    _methods = ("append_frame", "evict_frames", "execute_deferred_eviction", "rollback_last_frame", "compute_attention",
                "reset", "get_cache_stats", "build_visible_page_table", "compute_last_page_len")

    def __init__(self, manager):
        object.__setattr__(self, "_m", manager)

    def __getattr__(self, name):
        if name in self._methods or name in ("_skip_append", "_defer_eviction", "num_blocks", "tokens_per_frame", "frame_count",
                                              "kv_caches", "page_size", "scale_frames", "sliding_window", "dtype", "device",
                                              "num_frames"):
            return getattr(self._m, name)
        raise AttributeError(name)

    def __setattr__(self, name, value):
        setattr(self._m, name, value)


@pytest.mark.parametrize("drive", ["step", "reference_calls"])
def test_stream_at_the_reference_defaults(drive):
    """104 frames: the 8 anchor frames, then 96 streamed ones of which every seventh only reads
    the cache - 82 streamed keyframes, so the window of 64 has been full and evicting for 18
    keyframes at the end.  ``step``: the manager's fused step.  ``reference_calls``: the block's
    attention module driving the reference's methods one by one, non-keyframes as defer / append /
    attend / roll back."""
    from lingbot_map_amd import HipPagedAttention, HipPagedKVCacheManager
    from oracle.page_policy import PagePolicy
    from oracle.sdpa_cache import PagedStreamOracle
    dev = torch.device("cuda:0")
    m = HipPagedKVCacheManager(1, ANCHOR + WINDOW + 16, T, H, D, torch.bfloat16, dev, num_special_tokens=N_SP,
                               scale_frames=ANCHOR, sliding_window=WINDOW, max_total_frames=MAX_TOTAL)
    assert m.layout == "two_stream" and m.page_size == T - N_SP == 999
    pol = PagePolicy(T, N_SP, None, ANCHOR, WINDOW, MAX_TOTAL)
    assert pol.page_size == 999 and m.max_num_pages == pol.max_num_pages
    orc = PagedStreamOracle(pol, H, D, torch.bfloat16)
    attn = HipPagedAttention(H * D, H, kv_cache_sliding_window=WINDOW, kv_cache_scale_frames=ANCHOR)
    surface = ReferenceSurfaceOnly(m)
    g = torch.Generator().manual_seed(6)
    n_frames, keyframes, checked = 104, 0, []
    for f in range(n_frames):
        keyframe = f < ANCHOR or (f - ANCHOR) % 7 != 3
        q, k, v = (torch.randn(T, H, D, generator=g).to(torch.bfloat16) for _ in range(3))
        if drive == "step":
            out = m.step(0, q.to(dev), k.to(dev), v.to(dev), keyframe=[keyframe])
        else:
            m._skip_append = not keyframe
            out = attn.stream_attend(surface, 0, q.to(dev), k.to(dev), v.to(dev))
            m._skip_append = False
        # the oracle: keyframe = append + evict; a non-keyframe leaves no trace
        want = f in (0, ANCHOR - 1, ANCHOR, 40) or f >= n_frames - 3 or (not keyframe and f > 90)
        if keyframe:
            orc.append_frame(k, v)
            pol.evict_frames(ANCHOR, WINDOW)
            keyframes += 1
            ref = orc.compute_attention(q) if want else None
        else:
            ref = orc.step(q, k, v, keyframe=False) if want else None
        assert m.build_visible_page_table(0) == pol.build_visible_page_table(), f
        assert m.compute_last_page_len(0) == pol.compute_last_page_len(), f
        assert m.frame_count[0] == pol.frame_count == keyframes
        if ref is not None:
            check(out, ref, f"frame {f} ({'key' if keyframe else 'read-only'})")
            checked.append((f, keyframe, sum(pol.build_visible_page_lens())))
    st = m.get_cache_stats(0)
    assert st["scale_pages"] == ANCHOR and st["live_pages"] == WINDOW and st["special_tokens"] == N_SP * keyframes
    assert keyframes - ANCHOR >= 80 and m.device_header()["error"] == 0
    # the steady state was among the checked frames: 72 frames of 999 patches + every keyframe's specials
    assert max(n for _, _, n in checked) == (ANCHOR + WINDOW) * 999 + N_SP * keyframes >= 72_000
    assert any(not kf for f, kf, _ in checked if f > 90)


def test_anchor_pass_of_eight_frames_at_full_size():
    """Phase 1 of the streaming model at the reference's defaults (attention.py:475-511,
    demo.py:367): 8 frames of 1005 tokens arrive in one call, attend to one another (8,040 x 8,040
    per stream - the split-KV kernel over the stream's own rows) and are appended frame by frame.
    Two streams side by side.  Then one more frame is streamed and must see the 8 anchor frames
    and itself.  Reference: the oracle's producer (the reference's bf16 rounding sequence) on the
    module's own qkv projection, fp32 SDPA per stream, and ``PagedStreamOracle`` for the cache."""
    from lingbot_map_amd import HipPagedAttention, HipPagedKVCacheManager, RotaryPositionEmbedding3D
    from oracle.page_policy import PagePolicy
    from oracle.prepare_qkv import prepare_qkv
    from oracle.sdpa_cache import PagedStreamOracle, sdpa_nhd
    torch.manual_seed(8)
    dev = torch.device("cuda:0")
    B, S, dim = 2, ANCHOR, H * D
    rope3d = RotaryPositionEmbedding3D(D)
    attn = HipPagedAttention(dim, H, qk_norm=True, rope=rope3d, kv_cache_sliding_window=WINDOW,
                             kv_cache_scale_frames=ANCHOR).to(dev, torch.bfloat16).eval()
    with torch.no_grad():
        for norm in (attn.q_norm, attn.k_norm):
            norm.weight.add_(0.2 * torch.randn_like(norm.weight))
            norm.bias.add_(0.1 * torch.randn_like(norm.bias))
    attn.proj = torch.nn.Identity()          # compare the attention itself
    m = HipPagedKVCacheManager(1, ANCHOR + WINDOW + 16, T, H, D, torch.bfloat16, dev, num_special_tokens=N_SP,
                               scale_frames=ANCHOR, sliding_window=WINDOW, max_total_frames=64, num_streams=B)
    pols = [PagePolicy(T, N_SP, None, ANCHOR, WINDOW, 64, page_base=b * m.max_num_pages) for b in range(B)]
    orcs = [PagedStreamOracle(p, H, D, torch.bfloat16) for p in pols]
    qn = (attn.q_norm.weight.detach().cpu(), attn.q_norm.bias.detach().cpu())
    kn = (attn.k_norm.weight.detach().cpu(), attn.k_norm.bias.detach().cpu())

    def reference_qkv(x, table):
        """q, k, v ``[B, n, H, D]`` bf16 from the module's own projection of ``x``."""
        with torch.no_grad():
            qkv = attn.qkv(x).cpu()
        return [torch.stack(t) for t in zip(*[prepare_qkv(qkv[b], H, D, qn, kn, table.cpu()) for b in range(B)])]

    with torch.no_grad():
        x = torch.randn(B, S * T, dim, device=dev).to(torch.bfloat16)
        table = rope3d(ppf=S, pph=27, ppw=37, patch_start_idx=N_SP, device=dev, f_start=0, f_end=S)
        out = attn(x, pos=table, enable_3d_rope=True, kv_cache=m, global_idx=0, num_frames=S)
        rq, rk, rv = reference_qkv(x, table)
        for b in range(B):
            check(out[b].reshape(S * T, H, D), sdpa_nhd(rq[b], rk[b], rv[b]), f"anchor pass, stream {b}")
            for f in range(S):
                orcs[b].append_frame(rk[b, f * T:(f + 1) * T], rv[b, f * T:(f + 1) * T])
                pols[b].evict_frames(ANCHOR, WINDOW)
            assert m.build_visible_page_table(0, stream=b) == pols[b].build_visible_page_table()
            assert m.compute_last_page_len(0, stream=b) == pols[b].compute_last_page_len()
            # what the pass left in the pool is what the oracle cached: v exactly; k equal except where
            # the fp32 sums of the q/k LayerNorm, taken in another order, moved a normalised value (up to
            # about 4 in magnitude: a bf16 step of 2^-5) by one step before the rotation
            ids, lens = pols[b].build_visible_page_table(), pols[b].build_visible_page_lens()
            pool = m.kv_caches[0].cpu()
            differ = total = 0
            for p, n in zip(ids, lens):
                assert torch.equal(pool[p, 1, :n], orcs[b].pool[p, 1, :n])
                dk = (pool[p, 0, :n].float() - orcs[b].pool[p, 0, :n].float()).abs()
                assert dk.max().item() <= 2 ** -5, dk.max().item()
                differ, total = differ + int((dk > 0).sum()), total + dk.numel()
            assert differ < 1e-3 * total, (differ, total)
        assert m.frame_count == [S]
        # one streamed frame on top
        x1 = torch.randn(B, T, dim, device=dev).to(torch.bfloat16)
        table1 = rope3d(ppf=1, pph=27, ppw=37, patch_start_idx=N_SP, device=dev, f_start=S, f_end=S + 1)
        out1 = attn(x1, pos=table1, enable_3d_rope=True, kv_cache=m, global_idx=0, num_frames=1)
        q1, k1, v1 = reference_qkv(x1, table1)
        for b in range(B):
            check(out1[b].reshape(T, H, D), orcs[b].step(q1[b], k1[b], v1[b], keyframe=True), f"first streamed frame, stream {b}")
    assert m.device_header()["error"] == 0
