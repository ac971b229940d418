"""Pins for oracle/sdpa_cache.py (CPU only): the arithmetic against closed forms and a
float64 three-loop softmax, and the three cache formulations against each other."""
import math

import numpy as np
import pytest
import torch

from oracle.page_policy import LAYOUT_FRAME_PAGES, LAYOUT_TWO_STREAM, PagePolicy, is_keyframe
from oracle.sdpa_cache import (DictCacheOracle, PagedStreamOracle, attention_with_lse, gather_paged,
                               merge_splits, naive_attention_f64, sdpa_nhd)


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def test_sdpa_matches_float64_loops():
    q, k, v = rnd(5, 2, 8, seed=1), rnd(11, 2, 8, seed=2), rnd(11, 2, 8, seed=3)
    ref = naive_attention_f64(q.numpy(), k.numpy(), v.numpy())
    got = sdpa_nhd(q, k, v).double().numpy()
    assert np.abs(got - ref).max() < 2e-6
    # a dropped 1/sqrt(D) or a transposed operand must fail this check
    wrong = torch.softmax(torch.einsum("qhd,khd->hqk", q, k), -1)
    wrong = torch.einsum("hqk,khd->qhd", wrong, v).double().numpy()
    assert np.abs(wrong - ref).max() > 1e-2


def test_single_kv_token_returns_v():
    q, k, v = rnd(4, 3, 16, seed=4), rnd(1, 3, 16, seed=5), rnd(1, 3, 16, seed=6)
    out = sdpa_nhd(q, k, v)
    assert torch.allclose(out, v.expand(4, 3, 16), atol=1e-6)


def test_identical_keys_average_values():
    q, v = rnd(3, 2, 8, seed=7), rnd(9, 2, 8, seed=8)
    k = rnd(1, 2, 8, seed=9).expand(9, 2, 8).contiguous()
    out = sdpa_nhd(q, k, v)
    assert torch.allclose(out, v.mean(0, keepdim=True).expand(3, 2, 8), atol=1e-6)


def test_permutation_invariance_and_split_merge():
    q, k, v = rnd(6, 2, 16, seed=10), rnd(40, 2, 16, seed=11), rnd(40, 2, 16, seed=12)
    base = sdpa_nhd(q, k, v)
    perm = torch.randperm(40, generator=torch.Generator().manual_seed(13))
    assert torch.allclose(sdpa_nhd(q, k[perm], v[perm]), base, atol=1e-6)
    o1, l1 = attention_with_lse(q, k[:13], v[:13])
    o2, l2 = attention_with_lse(q, k[13:], v[13:])
    merged = merge_splits([o1, o2], [l1, l2])
    assert torch.allclose(merged.float(), base, atol=1e-6)


def test_bf16_inputs_fp32_math():
    q, k, v = (rnd(8, 2, 64, seed=s, dtype=torch.bfloat16) for s in (14, 15, 16))
    out = sdpa_nhd(q, k, v)
    assert out.dtype == torch.bfloat16
    ref = naive_attention_f64(q.float().numpy(), k.float().numpy(), v.float().numpy())
    assert np.abs(out.float().numpy() - ref).max() < 1e-2


def token_ids(frame, tokens, heads=1, dim=2):
    """K and V whose entries name (frame, token) so that sets of tokens can be compared."""
    base = torch.arange(tokens, dtype=torch.float32).view(tokens, 1, 1).expand(tokens, heads, dim)
    return (frame * 1000 + base).clone(), (-(frame * 1000 + base)).clone()


@pytest.mark.parametrize("layout,page_size", [(LAYOUT_TWO_STREAM, None), (LAYOUT_TWO_STREAM, 4),
                                              (LAYOUT_FRAME_PAGES, 4), (LAYOUT_FRAME_PAGES, 16)])
@pytest.mark.parametrize("interval", [1, 3])
def test_paged_visible_set_equals_dict_cache_set(layout, page_size, interval):
    T, n_sp, scale, window = 23, 5, 2, 3
    pol = PagePolicy(T, n_sp, page_size, scale, window, max_total_frames=64, layout=layout)
    paged = PagedStreamOracle(pol, 1, 2)
    dic = DictCacheOracle(scale, window, n_sp)
    for f in range(40):
        k, v = token_ids(f, T)
        kf = is_keyframe(f, scale, interval)
        dk, dv = dic.visible(k, v, kf)
        if kf:
            paged.append_frame(k, v); pol.evict_frames(scale, window)
            pk, pv = gather_paged(paged.pool, pol.build_visible_page_table(), pol.build_visible_page_lens())
        else:
            pol._defer_eviction = True
            paged.append_frame(k, v)
            pk, pv = gather_paged(paged.pool, pol.build_visible_page_table(), pol.build_visible_page_lens())
            pol.rollback_last_frame(); pol._defer_eviction = False
        assert sorted(pk[:, 0, 0].tolist()) == sorted(dk[:, 0, 0].tolist()), f"frame {f}"
        assert sorted(pv[:, 0, 0].tolist()) == sorted(dv[:, 0, 0].tolist())
        assert len(pk) == pol.visible_tokens() or not kf


def test_camera_only_and_no_memory_sets():
    T, n_sp, scale, window = 11, 3, 1, 2
    for kw in ({"camera_only": True}, {"cross_frame_special": False}):
        pol = PagePolicy(T, n_sp, 4, scale, window, max_total_frames=32, layout=LAYOUT_FRAME_PAGES)
        paged = PagedStreamOracle(pol, 1, 2)
        dic = DictCacheOracle(scale, window, n_sp, **kw)
        for f in range(12):
            k, v = token_ids(f, T)
            dk, _ = dic.visible(k, v)
            paged.append_frame(k, v); pol.evict_frames(scale, window, **kw)
            pk, _ = gather_paged(paged.pool, pol.build_visible_page_table(), pol.build_visible_page_lens())
            assert sorted(pk[:, 0, 0].tolist()) == sorted(dk[:, 0, 0].tolist())


def test_stream_outputs_agree_fp32_config1_shape_reduced():
    # config-1 semantics on a reduced frame: every frame attends to all cached frames and itself
    T, H, D, n_sp = 40, 2, 64, 5
    pol = PagePolicy(T, n_sp, 16, scale_frames=1, sliding_window=16, max_total_frames=16, layout=LAYOUT_FRAME_PAGES)
    paged = PagedStreamOracle(pol, H, D)
    dic = DictCacheOracle(1, 16, n_sp)
    g = torch.Generator().manual_seed(0)
    ks, vs = [], []
    for f in range(8):
        q, k, v = (torch.randn(T, H, D, generator=g) / 8 for _ in range(3))
        ks.append(k); vs.append(v)
        a = paged.step(q, k, v)
        b = dic.step(q, k, v)
        c = sdpa_nhd(q, torch.cat(ks), torch.cat(vs))
        assert (a - b).abs().max() < 1e-5 and (a - c).abs().max() < 1e-5
