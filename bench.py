"""Benchmark of the streaming paged-KV attention hot path on one MI355X.

A step is one streamed frame at 518x378 through the hot path of all global blocks: one
index-kernel launch (allocate, evict, visible rows) and, per block, the paged K/V append
and the paged attention of the frame's 1004 query tokens over 1 anchor + 16 window frames
(17,068 KV tokens, 16-token pages, 16 heads, head_dim 64, bf16).  Inputs are synthetic
N(0,1) tensors already resident in HBM.  Prints one JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--blocks 24]
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "lingbot-map_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

T, N_SPECIAL, H, D, PAGE = 1004, 5, 16, 64, 16
ANCHOR, WINDOW = 1, 16
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0
# HBM bytes of one lbm_attn_run at this workload - the main kernel AND the combine kernel that
# merges its split-KV partial results - from rocprofv3 --pmc FETCH_SIZE (x2.0, the factor a
# 256 MiB plain copy gives) and WRITE_SIZE (x1.0), in KiB per dispatch
# (profiles/attention_config2_hbm_traffic.md): main ATTN_MAIN_KIB, combine ATTN_COMBINE_KIB
ATTN_MAIN_KIB = (35503.5, 20080.0)       # (FETCH_SIZE, WRITE_SIZE) of lbm_attn_bf16_d64_kernel
ATTN_COMBINE_KIB = (8313.9, 2008.0)      # of lbm_attn_combine_bf16_kernel
ATTN_TRAFFIC_BYTES = ((ATTN_MAIN_KIB[0] + ATTN_COMBINE_KIB[0]) * 2.0 + ATTN_MAIN_KIB[1] + ATTN_COMBINE_KIB[1]) * 1024.0
METRIC = "frames/sec streaming @518x378 (1 GPU); attention TFLOPS & % bf16 MFMA peak"


def kernel_time_ms(fn, iters: int, torch) -> float:
    """Average GPU time of one fn() launch in ms for kernels shorter than the host's launch
    overhead: `iters` launches are captured into one HIP graph, the graph is replayed and
    timed with a HIP event pair on the launch stream, so the launches run back to back."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()  # warm up outside capture
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(iters):
                fn()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        graph.replay()
        side.synchronize()
        start.record(side)
        for _ in range(4):
            graph.replay()
        stop.record(side)
        stop.synchronize()
    torch.cuda.current_stream().wait_stream(side)
    return start.elapsed_time(stop) / (4 * iters)


def event_time_ms(fn, iters: int, torch) -> float:
    """Average duration of fn() in ms from one HIP event pair on the launch stream."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def attention_shapes(torch) -> list:
    """One lbm_attn_run at the attention shapes of the other configurations (synthetic bf16 pools and
    row tables built here; HIP events around 100 launches after 100 warm-up launches)."""
    import ctypes as C
    from lingbot_map_amd import _native as N
    dev = torch.device("cuda:0")

    def run(name, kvs, tail=False, shuffle_seed=None):
        ns = len(kvs)
        g = torch.Generator(device=dev).manual_seed(0)
        q = torch.randn(ns * T, H, D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        n_pages = sum(-(-kv // PAGE) for kv in kvs)
        pool = torch.randn(n_pages, 2, PAGE, H, D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        order = torch.arange(n_pages)
        if shuffle_seed is not None:   # cached pages scattered over the pool
            order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(shuffle_seed))
        rows, begin, off, base = [], [], 0, 0
        for b, kv in enumerate(kvs):
            begin.append(off)
            r = torch.arange(kv)
            rr = order[r // PAGE + base] * 2 * PAGE + r % PAGE
            if tail:   # the frame's own K/V, not in the pool (entry -1 - row)
                rr[-T:] = -1 - (b * T + torch.arange(T))
            rows.append(rr.to(torch.int32))
            off += kv
            base += -(-kv // PAGE)
        kv_rows = torch.cat(rows).to(dev)
        streams = (N.AttnStream * ns)(*[N.AttnStream(b * T, T, begin[b], kvs[b]) for b in range(ns)])
        need = int(N.lib.lbm_attn_workspace_bytes(streams, ns, H, D))
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
        out = torch.empty_like(q)
        own = q if tail else None
        vp = lambda t: None if t is None else C.c_void_p(t.data_ptr())

        def launch():   # on whatever stream is current (the timing helpers launch on a stream of their own)
            N.check(N.lib.lbm_attn_run(vp(q), vp(pool), vp(out), vp(own), vp(own), vp(kv_rows), streams, ns, H, D, PAGE,
                                       N.DTYPE_BF16, 1.0 / math.sqrt(D), vp(ws), ws.numel(),
                                       C.c_void_p(torch.cuda.current_stream().cuda_stream)))

        for _ in range(100):
            launch()
        ms = event_time_ms(launch, 100, torch)
        if ms < 0.04:   # shorter than the host's launch cost: time back-to-back launches of a HIP graph instead
            ms = kernel_time_ms(launch, 50, torch)
        flop = 4.0 * T * sum(kvs) * H * D
        assert torch.isfinite(out.float()).all()
        return {"shape": name, "kv_tokens": kvs, "avg_launch_us": ms * 1e3, "tflops": flop / (ms * 1e-3) * 1e-12,
                "frac": flop / (ms * 1e-3) * 1e-12 / PEAK_BF16_TFLOPS}

    return [
        run("config 3: 67,068 tokens, pages in shuffled order", [67068], shuffle_seed=2),
        run("config 4 non-keyframe: 17,068 cached + the frame's own 1,004", [18072], tail=True),
        run("config 5: four streams, 5,020 / 9,036 / 17,068 / 17,068", [5020, 9036, 17068, 17068]),
        run("frame block: 1,004 x 1,004, no cache", [1004], tail=True),
    ]


def config3_stream(torch) -> dict:
    """Configuration 3 as a stream: one global block's cache after 10,000 frames (1 anchor + 16 window frames and
    9,983 evicted frames that kept their 5 special tokens in place: 66,983 visible tokens over 11,054 pages), then
    streamed keyframe steps on it.  Reports the table step alone (allocate + evict + compact + the 268 KB row table
    with its 9,983 memory frames) and a whole step of the block (table step + paged append + attention)."""
    from lingbot_map_amd import HipPagedKVCacheManager
    dev = torch.device("cuda:0")
    frames = 10000
    m = HipPagedKVCacheManager(1, ANCHOR + WINDOW + 16, T, H, D, torch.bfloat16, dev, num_special_tokens=N_SPECIAL,
                               scale_frames=ANCHOR, sliding_window=WINDOW, max_total_frames=frames + 64, page_size=PAGE,
                               layout="frame_pages")
    g = torch.Generator(device=dev).manual_seed(2)
    q, k, v = (torch.randn(T, H, D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(3))
    for _ in range(frames):
        m.append_frame(0, k, v)
        m.evict_frames(0, ANCHOR, WINDOW)
    kv = (ANCHOR + WINDOW) * T + N_SPECIAL * (frames - ANCHOR - WINDOW)
    m._plan(0, [False])
    assert m._plan_tokens[0][0] == kv == 66983
    ops = m._ops([{"ops": 16, "expect_kv_tokens": kv}])
    plan_ms = kernel_time_ms(lambda: m._tables_step(0, ops, kv_rows=True), 50, torch)
    for _ in range(5):
        m.step(0, q, k, v, keyframe=[True])
    step_ms = event_time_ms(lambda: m.step(0, q, k, v, keyframe=[True]), 20, torch)
    m._plan(0, [False])   # every visible row in the pool again (a step's table names its new frame by the caller's rows)
    attn_ms = event_time_ms(lambda: m._attend_planned(0, q, None, None), 50, torch)
    m.check_device_errors()
    kv_now = m._plan_tokens[0][0]
    flop = 4.0 * T * kv_now * H * D
    return {"kv_tokens": kv_now, "memory_frames": frames + 25 - ANCHOR - WINDOW, "tables_plan_us": plan_ms * 1e3,
            "block_step_us": step_ms * 1e3, "attention_us": attn_ms * 1e3,
            "attention_tflops": flop / (attn_ms * 1e-3) * 1e-12,
            "what": "one block: keyframe step = table step (allocate, evict, compact, row table) + paged append + attention "
                    "over anchor + window + trajectory memory; tables_plan_us is the row-table plan alone"}


def hbm_kernels_4_streams(torch) -> dict:
    """The three HBM-bound kernels at config 5's batch (four streams in one launch, 4,016 rows):
    the single-stream launches of 8-13 MB are as much launch ramp as stream."""
    import ctypes as C
    from lingbot_map_amd import HipPagedKVCacheManager
    from lingbot_map_amd import _native as N
    dev = torch.device("cuda:0")
    B = 4
    g = torch.Generator(device=dev).manual_seed(6)
    rnd = lambda *shape: torch.randn(*shape, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    m = HipPagedKVCacheManager(1, 8, T, H, D, torch.bfloat16, dev, num_special_tokens=N_SPECIAL, scale_frames=1,
                               sliding_window=2, max_total_frames=16, page_size=PAGE, layout="frame_pages", num_streams=B)
    k, v, qkv = rnd(B * T, H, D), rnd(B * T, H, D), rnd(B * T, 3 * H * D)
    m.append_frame(0, k, v)     # leaves the rows of one frame per stream in the append plan
    vp = lambda t: C.c_void_p(t.data_ptr())
    ln = [torch.rand(D, generator=g, device=dev) + 0.5 for _ in range(4)]
    ang = torch.rand(B * T, D // 2, generator=g, device=dev) * 6.283185
    cs = torch.stack([ang.cos(), ang.sin()], dim=-1).contiguous()
    q_out = torch.empty(B * T, H, D, dtype=torch.bfloat16, device=dev)
    x, y = rnd(B * T, H * D), rnd(B * T, H * D)
    par = [torch.rand(H * D, generator=g, device=dev) + 0.5 for _ in range(3)]
    outs = [torch.empty_like(x) for _ in range(2)]
    stream = lambda: m._stream_handle()
    fns = {
        "append": (lambda: m._scatter(0, m._append_rows[0], k, v), 2 * 2 * B * T * H * D * 2),
        "qkv_prepare": (lambda: N.check(N.lib.lbm_qkv_prepare(
            vp(qkv), N.DTYPE_BF16, vp(ln[0]), vp(ln[1]), vp(ln[2]), vp(ln[3]), 1e-5, 1.0, vp(cs), N.ROPE_INTERLEAVED, vp(q_out),
            None, None, N.DTYPE_BF16, vp(m.kv_caches[0]), vp(m._append_rows[0]), B * T, H, D, PAGE, stream())),
            6 * B * T * H * D * 2 + cs.numel() * 4),
        "residual_norm": (lambda: N.check(N.lib.lbm_residual_norm(
            vp(x), vp(y), N.DTYPE_BF16, vp(par[0]), vp(par[1]), vp(par[2]), 1e-5, vp(outs[0]), vp(outs[1]), B * T, H * D,
            stream())), 4 * B * T * H * D * 2),
    }
    res = {}
    for name, (fn, nbytes) in fns.items():
        ms = kernel_time_ms(fn, 100, torch)
        gbps = nbytes / (ms * 1e-3) * 1e-9
        res[name] = {"bytes_per_launch": nbytes, "avg_launch_us": ms * 1e3, "achieved": gbps, "unit": "GB/s",
                     "frac": gbps / PEAK_HBM_GBPS}
    assert m.device_header()["error"] == 0
    return res


def camera_head_cache(torch) -> dict:
    """The camera head's cache traffic of one streamed frame (lingbot_map/heads/camera_head.py:296-346,
    lingbot_map/layers/attention.py:224-349): 4 refinement iterations x 4 trunk blocks, each with
    its own cache of one 16 x 128 fp32 token per frame, nothing evicted.  One manager with 16
    blocks holds them; a frame is 16 x (append + attend).  Beside it the reference's scheme in
    plain PyTorch on the same GPU: concatenate the new token to the block's K and V, clone
    both, SDPA with an all-true mask."""
    from lingbot_map_amd import HipPagedKVCacheManager
    dev = torch.device("cuda:0")
    Hc, Dc, blocks, cached, timed = 16, 128, 16, 300, 50
    m = HipPagedKVCacheManager(blocks, cached + timed + 8, 1, Hc, Dc, torch.float32, dev, num_special_tokens=0,
                               scale_frames=8, sliding_window=cached + timed, max_total_frames=cached + timed + 8,
                               force_fp32=True, page_size=16, layout="frame_pages")
    g = torch.Generator(device=dev).manual_seed(8)
    qkv = [torch.randn(1, Hc, Dc, generator=g, device=dev) for _ in range(3)]
    dict_k = [torch.randn(1, Hc, cached, 1, Dc, generator=g, device=dev) for _ in range(blocks)]
    dict_v = [torch.randn(1, Hc, cached, 1, Dc, generator=g, device=dev) for _ in range(blocks)]

    def frame_hip():
        for b in range(blocks):
            out = m.step(b, qkv[0], qkv[1], qkv[2], keyframe=[True], cross_frame_special=False)
        return out

    def frame_dict():
        q = qkv[0].permute(1, 0, 2)[None]                        # [1, H, 1, D]
        for b in range(blocks):
            dict_k[b] = torch.cat((dict_k[b], qkv[1].view(1, Hc, 1, 1, Dc)), dim=2)
            dict_v[b] = torch.cat((dict_v[b], qkv[2].view(1, Hc, 1, 1, Dc)), dim=2)
            k = dict_k[b].clone().reshape(1, Hc, -1, Dc)
            v = dict_v[b].clone().reshape(1, Hc, -1, Dc)
            mask = torch.ones(1, 1, 1, k.shape[2], dtype=torch.bool, device=dev)
            out = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask)
        return out

    for _ in range(cached):
        frame_hip()
    res = {}
    for name, fn in (("hip_paged", frame_hip), ("torch_dict_cache", frame_dict)):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(timed - 5):
            out = fn()
        torch.cuda.synchronize()
        res[name + "_us_per_frame"] = (time.perf_counter() - t0) / (timed - 5) * 1e6
        assert torch.isfinite(out).all()
    assert m.device_header()["error"] == 0
    res["what"] = (f"{blocks} caches x (append one token + attend to ~{cached + timed // 2} cached tokens), 16 heads of 128, fp32, "
                   "wall clock per frame including the host's launches")
    # the same attention after 10,000 frames (the head never evicts): one launch, K/V read once
    del m
    long_frames = 10000
    ml = HipPagedKVCacheManager(1, long_frames + 16, 1, Hc, Dc, torch.float32, dev, num_special_tokens=0, scale_frames=8,
                                sliding_window=long_frames + 8, max_total_frames=long_frames + 16, force_fp32=True,
                                page_size=16, layout="frame_pages")
    for _ in range(long_frames):
        ml.append_frame(0, qkv[1], qkv[2])
    ml._plan(0, [False])
    for _ in range(10):
        ml._attend_planned(0, qkv[0], None, None)
    ms = event_time_ms(lambda: ml._attend_planned(0, qkv[0], None, None), 50, torch)
    nbytes = long_frames * Hc * Dc * 4 * 2
    res["attend_10000_frames"] = {"avg_launch_us": ms * 1e3, "bytes_per_launch": nbytes, "bound": "hbm",
                                  "achieved": nbytes / (ms * 1e-3) * 1e-9, "unit": "GB/s",
                                  "frac": nbytes / (ms * 1e-3) * 1e-9 / PEAK_HBM_GBPS,
                                  "what": "one query token over 10,000 cached tokens (few-query fp32 kernels: chunked KV + merge)"}
    return res


def config1(torch) -> dict:
    """Config 1, the CPU-runnable parity case: fp32, 8 frames of 1004 tokens, Q, K, V =
    randn / 8 with seed 0, frame i attends to frames 0..i (148.6 GFLOP in all).  The oracle's
    SDPA on the host cores beside the fp32 HIP kernel on the same inputs, and their largest
    difference."""
    from lingbot_map_amd import HipPagedKVCacheManager
    from oracle.sdpa_cache import sdpa_nhd
    torch.manual_seed(0)
    frames = 8
    qkv = [[torch.randn(T, H, D) / 8 for _ in range(3)] for _ in range(frames)]
    dev = torch.device("cuda:0")
    dq = [[t.to(dev) for t in f] for f in qkv]

    def cpu():
        outs = []
        for i in range(frames):
            k = torch.cat([f[1] for f in qkv[:i + 1]])
            v = torch.cat([f[2] for f in qkv[:i + 1]])
            outs.append(sdpa_nhd(qkv[i][0], k, v))
        return outs

    def gpu():
        m.reset()
        outs = []
        for i in range(frames):
            outs.append(m.step(0, dq[i][0], dq[i][1], dq[i][2], keyframe=[True]))
        return outs

    m = HipPagedKVCacheManager(1, 32, T, H, D, torch.float32, dev, num_special_tokens=N_SPECIAL, scale_frames=1,
                               sliding_window=16, max_total_frames=32, force_fp32=True, page_size=PAGE, layout="frame_pages")
    cpu()
    t0 = time.perf_counter()
    ref = cpu()
    t_cpu = time.perf_counter() - t0
    gpu()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    got = gpu()
    torch.cuda.synchronize()
    t_gpu = time.perf_counter() - t0
    err = max((a.cpu() - b).abs().max().item() for a, b in zip(got, ref))
    flops = sum(4.0 * T * (i + 1) * T * H * D for i in range(frames))
    # the attention launch of the last frame alone (1004 queries x 8032 cached tokens)
    m._plan(0, [False])
    for _ in range(20):
        m._attend_planned(0, dq[-1][0], None, None)
    k_ms = event_time_ms(lambda: m._attend_planned(0, dq[-1][0], None, None), 50, torch)
    k_flops = 4.0 * T * frames * T * H * D
    return {"cpu_ms": t_cpu * 1e3, "cpu_gflops": flops / t_cpu * 1e-9, "gpu_ms": t_gpu * 1e3,
            "gpu_gflops": flops / t_gpu * 1e-9, "max_abs_diff": err, "tolerance": 1e-5,
            "kernel": {"name": "lbm_attn_f32_kernel<64>", "bound": "mfma", "achieved": k_flops / (k_ms * 1e-3) * 1e-12,
                       "peak": 157.3, "unit": "TFLOP/s", "frac": k_flops / (k_ms * 1e-3) * 1e-12 / 157.3,
                       "avg_launch_us": k_ms * 1e3, "flop_per_launch": k_flops,
                       "what": "attention of frame 8 (1004 x 8032 tokens), HIP events around 50 launches after 20 warm-up launches"},
            "what": "8 frames, fp32, every frame attends to all frames so far (tables step + append + fp32 MFMA attention per frame, wall clock)"}


def cpu_baseline(torch, kv_tokens: int, blocks: int) -> dict:
    """The reference SDPA arithmetic (dense gather of the visible pages, then
    F.scaled_dot_product_attention) as restated by the oracle, on the host cores."""
    from oracle.sdpa_cache import gather_paged, sdpa_nhd
    g = torch.Generator().manual_seed(1)
    frames = ANCHOR + WINDOW
    ppf = -(-T // PAGE)
    pool = torch.randn(frames * ppf, 2, PAGE, H, D, generator=g).to(torch.bfloat16)
    ids = list(range(frames * ppf))
    lens = ([PAGE] * (ppf - 1) + [T - (ppf - 1) * PAGE]) * frames
    q = torch.randn(T, H, D, generator=g).to(torch.bfloat16)
    assert sum(lens) == kv_tokens

    def one():
        k, v = gather_paged(pool, ids, lens)
        return sdpa_nhd(q, k, v)

    for _ in range(2):
        one()
    times = []
    while len(times) < 15 or (sum(times) < 10.0 and len(times) < 400):   # about 10 s of host work
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    flops = 4.0 * T * kv_tokens * H * D
    c1 = config1(torch)
    return {
        "config1_fp32": c1,
        "value": 1.0 / (t * blocks), "unit": "frames/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"2 warm-up + {len(times)} timed layer-steps ({sum(times):.1f} s) of gather + SDPA (q {T} x kv {kv_tokens}, {H} heads, "
                  f"bf16 storage, fp32 math), median {t * 1e3:.1f} ms = {flops / t * 1e-9:.0f} GFLOP/s; "
                  f"frames/s = 1 / ({blocks} x median)",
    }


def aggregator_step(torch, blocks: int, steps: int, warmup: int, windows=(WINDOW,), keyframe_interval: int = 1) -> dict:
    """One streamed frame (a 3 x 378 x 518 image) of every stream through the product's aggregator
    shell (`lingbot_map_amd.HipAggregatorStream`): the image encoder's ViT-L trunk (patch
    convolution + 24 plain blocks + LayerNorm; lingbot_map/layers/vision_transformer.py:383-394)
    and `blocks` groups of (frame block, global block) (lingbot_map/aggregator/stream.py:415-529,
    base.py:575-606), special tokens first, group outputs concatenated, all at ViT-L size (dim
    1024, 16 heads, MLP 4096, LayerNorm, LayerScale; qk-norm and rotary embeddings in the
    aggregator blocks), random init, bf16.  The global blocks run the HIP cache path, every
    block's pre-attention producer and cache-less attention are HIP kernels too.  With one
    stream (one frame's rows per launch) a block is five launches of the package's own GEMM -
    qkv projection with norm1 folded in and the producer as its store, proj and fc2 with
    LayerScale + residual in theirs, fc1 with norm2 folded in and the GELU in its store - plus the
    attention; several streams batched take the same chain on their concatenated rows (the qkv
    projection and fc1 then on 256 x 256 tiles).  The patch convolution is PyTorch-ROCm.  The prediction
    heads are not part of the step.  `windows` holds one sliding window per stream: more than
    one entry runs that many independent streams as one ragged batch (a step is then one frame
    of every stream).  `keyframe_interval` > 1 caches every n-th frame only (config 4)."""
    from lingbot_map_amd import GraphedAggregator, HipAggregatorStream, PipelinedAggregator, set_skip_append
    dev = torch.device("cuda:0")
    torch.manual_seed(4)
    B = len(windows)
    # evicted frames leave no trajectory memory (as in the hot-path loop above), so the KV set
    # stays at 17,068 tokens per full window
    model = HipAggregatorStream(
        img_size=518, patch_size=14, embed_dim=H * D, depth=blocks, num_heads=H, mlp_ratio=4.0, num_register_tokens=4,
        qk_norm=True, init_values=0.01, patch_embed="vit", encoder_depth=24, enable_3d_rope=True, max_frame_num=156,
        kv_cache_sliding_window=list(windows) if B > 1 else windows[0], kv_cache_scale_frames=ANCHOR,
        kv_cache_cross_frame_special=False, use_scale_token=False, page_size=PAGE, layout="frame_pages",
        num_streams=B).to(dev, torch.bfloat16).eval()
    g = torch.Generator(device=dev).manual_seed(4)
    xs = [torch.rand(B, 1, 3, 378, 518, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(4)]
    selected = [4, 11, 17, blocks - 1] if blocks >= 24 else [blocks - 1]
    is_key = lambda i: keyframe_interval <= 1 or i % keyframe_interval == 0

    @torch.no_grad()
    def frame(i: int, keyframe: bool = True):
        set_skip_append(model.kv_cache_manager, not keyframe) if model.kv_cache_manager is not None else None
        return model(xs[i % len(xs)], selected_idx=selected)[0][-1]

    for i in range(ANCHOR + max(windows) + warmup):
        frame(i)
    assert model.kv_cache_manager.tokens_per_frame == T
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        out = frame(i, is_key(i))
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    set_skip_append(model.kv_cache_manager, False)
    assert torch.isfinite(out.float()).all()
    model.kv_cache_manager.check_device_errors()
    # the same frames replayed as HIP graphs (one for keyframes, one for read-only frames)
    graphed = GraphedAggregator(model, xs[0], selected_idx=selected)
    for i in range(3):
        graphed(xs[i % len(xs)], keyframe=is_key(i))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        out = graphed(xs[i % len(xs)], keyframe=is_key(i))
    torch.cuda.synchronize()
    dt_graph = (time.perf_counter() - t0) / steps
    assert torch.isfinite(out.float()).all()
    model.kv_cache_manager.check_device_errors()
    # one frame of look-ahead: the next frame's image encoder as a second branch of the graph that
    # takes the present frame through its frame and global blocks (same results, one call later)
    del graphed
    piped = PipelinedAggregator(model, xs[0], selected_idx=selected)
    piped.prime(xs[0])
    for i in range(3):
        piped(xs[(i + 1) % len(xs)], keyframe=is_key(i))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        out = piped(xs[(i + 1) % len(xs)], keyframe=is_key(i))
    torch.cuda.synchronize()
    dt_piped = (time.perf_counter() - t0) / steps
    assert torch.isfinite(out.float()).all()
    model.kv_cache_manager.check_device_errors()
    kv = " / ".join(str((ANCHOR + w) * T) for w in windows)
    return {"value": B / dt, "unit": "frames/s", "ms_per_step": dt * 1e3, "steps": steps, "streams": B,
            "keyframe_interval": keyframe_interval,
            "hip_graph": {"value": B / dt_graph, "unit": "frames/s", "ms_per_step": dt_graph * 1e3},
            "hip_graph_lookahead": {"value": B / dt_piped, "unit": "frames/s", "ms_per_step": dt_piped * 1e3,
                                    "what": "PipelinedAggregator: the image encoder of frame t + 1 and the frame and global "
                                            "blocks of frame t as two branches of one HIP graph; a frame's outputs arrive one "
                                            "call after its image, bit-equal to the plain replay"},
            "what": f"HipAggregatorStream: patch convolution + 24 encoder blocks + {blocks} x (frame block + global block), "
                    f"dim {H * D}, {H} heads, MLP {4 * H * D}, {B} stream(s), {T} tokens/frame, steady-state cache of {kv} "
                    f"KV tokens; the package's GEMM with fused LayerNorm / GELU / LayerScale + residual / producer for every linear"
                    ", HIP kernels for the cache path and every block's cache-less attention, PyTorch-ROCm for the patch "
                    "convolution; prediction heads excluded"}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--blocks", type=int, default=24)
    ap.add_argument("--streams", type=int, default=1, help="--mode aggregator: independent streams batched per step")
    ap.add_argument("--constant-kv", action="store_true",
                    help="--mode attention: every cached K and V element is 0.5 instead of N(0, 1) - the same instruction "
                         "stream on operands that switch no bits, to separate the kernel's cycle count from the clock "
                         "the chip sustains under it")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-aggregator", action="store_true",
                    help="skip the full aggregator-trunk step (frame + global blocks) timed after the hot path")
    ap.add_argument("--mode", choices=["full", "attention", "attention_frame", "attention_f32", "attention_f32_few", "append", "prepare", "residual", "tables", "copy", "linear", "aggregator"], default="full",
                    help="full = the benchmark line; attention/attention_frame (a frame block's 1004 x 1004 without cache)/attention_f32/attention_f32_few/append/prepare/residual/tables launch one kernel --steps "
                         "times on the steady-state cache (for rocprofv3 runs); copy = a plain 256 MiB "
                         "device copy, the known-size kernel the HBM counters are calibrated on")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this path is built and measured on ONE GPU; --gpus N with N > 1 is not supported "
                 "(independent streams would shard across GPUs without communication)")

    import torch
    from lingbot_map_amd import HipPagedKVCacheManager

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.mode == "copy":
        src = torch.full((256 << 20,), 3, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(args.warmup):
            dst.copy_(src)
        ms = event_time_ms(lambda: dst.copy_(src), args.steps, torch)
        print(json.dumps({"mode": "copy", "bytes_read": src.numel(), "bytes_written": dst.numel(),
                          "launches": args.steps, "avg_launch_us": ms * 1e3}))
        return
    if args.mode == "aggregator":
        # the aggregator step alone (eager, then replayed as HIP graphs): one stream, or with
        # --streams 4 configuration 5's four ragged streams
        windows = (WINDOW,) if args.streams == 1 else (4, 8, 16, 16)[:args.streams] if args.streams <= 4 else (WINDOW,) * args.streams
        print(json.dumps({"mode": "aggregator", "streams": args.streams,
                          "aggregator_step": aggregator_step(torch, args.blocks, 12, 3, windows=windows)}))
        return
    if args.mode == "linear":
        # the four linears of a block at one frame (1004 rows), two and four streams (2008, 4016 rows):
        # lbm_linear with its fused epilogue against the PyTorch-ROCm calls it replaces
        from lingbot_map_amd import _native as N
        import ctypes as C
        import torch.nn.functional as F
        vp = lambda t: None if t is None else C.c_void_p(t.data_ptr())
        g = torch.Generator(device=dev).manual_seed(5)
        rows = []
        for M in (1004, 2008, 4016):
            for name, K, Nn, epi in (("qkv", 1024, 3072, N.LINEAR_BIAS), ("proj + ls + residual", 1024, 1024, N.LINEAR_BIAS_RESIDUAL),
                                     ("fc1 + gelu", 1024, 4096, N.LINEAR_BIAS_GELU), ("fc2 + ls + residual", 4096, 1024, N.LINEAR_BIAS_RESIDUAL)):
                a = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
                w = (torch.randn(Nn, K, generator=g, device=dev) / K ** 0.5).to(torch.bfloat16)
                b = torch.randn(Nn, generator=g, device=dev).to(torch.bfloat16)
                gam = torch.rand(Nn, generator=g, device=dev).to(torch.bfloat16)
                res = torch.randn(M, Nn, generator=g, device=dev).to(torch.bfloat16)
                b32, g32 = b.float(), gam.float()
                out = torch.empty(M, Nn, dtype=torch.bfloat16, device=dev)
                residual = epi == N.LINEAR_BIAS_RESIDUAL
                stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
                ours = lambda: N.check(N.lib.lbm_linear(vp(a), vp(w), vp(b32), vp(g32) if residual else None,
                                                         vp(res) if residual else None, vp(out), M, Nn, K, epi, stream()))
                if epi == N.LINEAR_BIAS:
                    theirs = lambda: F.linear(a, w, b)
                elif epi == N.LINEAR_BIAS_GELU:
                    theirs = lambda: F.gelu(F.linear(a, w, b))
                else:
                    theirs = lambda: res + F.linear(a, w, b) * gam
                for _ in range(3):
                    ours(); theirs()
                t_ours, t_theirs = kernel_time_ms(ours, 50, torch) * 1e3, kernel_time_ms(theirs, 50, torch) * 1e3
                flop = 2.0 * M * K * Nn
                rows.append({"layer": name, "M": M, "K": K, "N": Nn, "lbm_linear_us": t_ours, "torch_us": t_theirs,
                             "lbm_linear_tflops": flop / t_ours * 1e-6, "torch_tflops": flop / t_theirs * 1e-6})
        # the chained forms at one frame's rows: row statistics out of the residual launches (fc2
        # with K split over two workgroups per tile), LayerNorm folded into the launch that follows
        chained = []
        M = 1004
        for name, K, Nn, epi, fold in (("qkv, norm1 folded in", 1024, 3072, N.LINEAR_BIAS, True),
                                       ("proj + ls + residual + row statistics", 1024, 1024, N.LINEAR_BIAS_RESIDUAL, False),
                                       ("fc1 + gelu, norm2 folded in", 1024, 4096, N.LINEAR_BIAS_GELU, True),
                                       ("fc2 + ls + residual + row statistics, K split", 4096, 1024, N.LINEAR_BIAS_RESIDUAL, False)):
            a = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
            w = (torch.randn(Nn, K, generator=g, device=dev) / K ** 0.5).to(torch.bfloat16)
            b32 = torch.randn(Nn, generator=g, device=dev)
            g32 = torch.rand(Nn, generator=g, device=dev)
            res = torch.randn(M, Nn, generator=g, device=dev).to(torch.bfloat16)
            out = torch.empty(M, Nn, dtype=torch.bfloat16, device=dev)
            stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
            if fold:
                tiles = 16
                xs = a.float().reshape(M, tiles, -1)
                mean = xs.mean(-1)
                stats = torch.stack([mean, ((xs - mean[..., None]) ** 2).sum(-1)], -1).contiguous()
                colsum = w.float().sum(1).contiguous()
                ln = N.RowNorm(stats.data_ptr(), colsum.data_ptr(), tiles, 1e-5)
                fn = lambda: N.check(N.lib.lbm_linear_norm(vp(a), ln, vp(w), vp(b32), None, None, vp(out), None, M, Nn, K, epi,
                                                           None, 0, stream()))
            else:
                tiles = N.lib.lbm_linear_stats_tiles(M, Nn)
                stats = torch.empty(M, tiles, 2, device=dev)
                need = N.lib.lbm_linear_workspace_bytes(M, Nn, K, epi)
                ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=dev)
                fn = lambda: N.check(N.lib.lbm_linear_norm(vp(a), None, vp(w), vp(b32), vp(g32), vp(res), vp(out), vp(stats), M, Nn, K,
                                                           epi, vp(ws) if need else None, need, stream()))
            for _ in range(3):
                fn()
            t = kernel_time_ms(fn, 50, torch) * 1e3
            chained.append({"layer": name, "M": M, "K": K, "N": Nn, "lbm_linear_norm_us": t, "tflops": 2.0 * M * K * Nn / t * 1e-6})
        # time against K at one shape: slope = the loop per 128 of K, intercept = launch, prologue, store
        sweep = []
        Nn = 3072
        for K in (256, 512, 1024, 2048, 4096):
            a = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
            w = (torch.randn(Nn, K, generator=g, device=dev) / K ** 0.5).to(torch.bfloat16)
            b = torch.randn(Nn, generator=g, device=dev).to(torch.bfloat16)
            b32 = b.float()
            out = torch.empty(M, Nn, dtype=torch.bfloat16, device=dev)
            stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
            ours = lambda: N.check(N.lib.lbm_linear(vp(a), vp(w), vp(b32), None, None, vp(out), M, Nn, K, N.LINEAR_BIAS, stream()))
            theirs = lambda: F.linear(a, w, b)
            for _ in range(3):
                ours(); theirs()
            sweep.append({"M": M, "N": Nn, "K": K, "lbm_linear_us": kernel_time_ms(ours, 50, torch) * 1e3,
                          "torch_us": kernel_time_ms(theirs, 50, torch) * 1e3})
        # the qkv projection with the producer as its store, form by form (what the q/k LayerNorm,
        # the rotary layouts and the pool copy add to the launch), one and four frames' rows
        forms = []
        K, Nn = 1024, 3 * H * D
        for M in (4 * T, T):
            a = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
            w = (torch.randn(Nn, K, generator=g, device=dev) / K ** 0.5).to(torch.bfloat16)
            b32 = torch.randn(Nn, generator=g, device=dev)
            tiles = 16
            xs = a.float().reshape(M, tiles, -1)
            mean = xs.mean(-1)
            stats = torch.stack([mean, ((xs - mean[..., None]) ** 2).sum(-1)], -1).contiguous()
            colsum = w.float().sum(1).contiguous()
            ln = N.RowNorm(stats.data_ptr(), colsum.data_ptr(), tiles, 1e-5)
            qk_norm = [torch.randn(D, generator=g, device=dev) for _ in range(4)]
            pairs = torch.randn(M, D // 2, 2, generator=g, device=dev)
            halves = torch.randn(M, D, 2, generator=g, device=dev)
            q, k, v = (torch.empty(M, H, D, dtype=torch.bfloat16, device=dev) for _ in range(3))
            pool = torch.empty((M + PAGE - 1) // PAGE + 1, 2, PAGE, H, D, dtype=torch.bfloat16, device=dev)
            t_idx = torch.arange(M, device=dev, dtype=torch.int32)
            pool_rows = (t_idx // PAGE * 2 * PAGE + t_idx % PAGE).contiguous()
            stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)

            def form(norm, table, layout, plain, pooled):
                nw = [vp(t) for t in qk_norm] if norm else [None] * 4
                return lambda: N.check(N.lib.lbm_qkv_linear_prepare_norm(
                    vp(a), ln, vp(w), vp(b32), M, K, nw[0], nw[1], nw[2], nw[3], 1e-5, 0.18, vp(table) if table is not None else None,
                    layout, vp(q), vp(k) if plain else None, vp(v) if plain else None, vp(pool) if pooled else None,
                    vp(pool_rows) if pooled else None, H, D, PAGE, stream()))
            for name, fn in (("no q/k norm, no rotary, plain q/k/v", form(False, None, N.ROPE_INTERLEAVED, True, False)),
                             ("q/k norm", form(True, None, N.ROPE_INTERLEAVED, True, False)),
                             ("interleaved rotary", form(False, pairs, N.ROPE_INTERLEAVED, True, False)),
                             ("interleaved rotary + q/k norm", form(True, pairs, N.ROPE_INTERLEAVED, True, False)),
                             ("half-split rotary + q/k norm", form(True, halves, N.ROPE_HALF_SPLIT, True, False)),
                             ("half-split rotary + q/k norm, K/V into pool pages only", form(True, halves, N.ROPE_HALF_SPLIT, False, True)),
                             ("half-split rotary + q/k norm, plain q/k/v and pool pages", form(True, halves, N.ROPE_HALF_SPLIT, True, True))):
                for _ in range(10):
                    fn()
                forms.append({"form": name, "M": M, "lbm_qkv_linear_prepare_norm_us": kernel_time_ms(fn, 50, torch) * 1e3})
        # weights that no cache holds (a model walks through far more weight bytes per frame than the
        # caches hold): the same launch on one weight matrix every time, on weights rotating through
        # 640 MB, and on the rotating weights with each launch told (lbm_linear_prefetch_hint) what
        # the launch after it will read
        cold = []
        M = T
        for name, Nn, K, epi in (("qkv", 3072, 1024, N.LINEAR_BIAS), ("proj", 1024, 1024, N.LINEAR_BIAS),
                                 ("fc1 + gelu", 4096, 1024, N.LINEAR_BIAS_GELU), ("fc2", 1024, 4096, N.LINEAR_BIAS)):
            copies = max(2, (640 << 20) // (Nn * K * 2))
            a = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
            ws = [(torch.randn(Nn, K, generator=g, device=dev) / K ** 0.5).to(torch.bfloat16) for _ in range(copies)]
            b32 = torch.randn(Nn, generator=g, device=dev)
            out = torch.empty(M, Nn, dtype=torch.bfloat16, device=dev)
            stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
            at = [0]

            def launch(rotate: bool, hint: bool):
                if rotate:
                    at[0] = (at[0] + 1) % copies
                if hint:
                    nxt = ws[(at[0] + 1) % copies]
                    N.check(N.lib.lbm_linear_prefetch_hint(vp(nxt), nxt.numel() * 2))
                N.check(N.lib.lbm_linear(vp(a), vp(ws[at[0]]), vp(b32), None, None, vp(out), M, Nn, K, epi, stream()))
            times = {}
            for label, rotate, hint in (("same_weights_us", False, False), ("rotating_weights_us", True, False),
                                        ("rotating_weights_hinted_us", True, True)):
                fn = lambda: launch(rotate, hint)
                for _ in range(3):
                    fn()
                times[label] = kernel_time_ms(fn, 100, torch) * 1e3
            cold.append({"layer": name, "M": M, "K": K, "N": Nn, "weight_copies": copies, **times})
            del ws
        print(json.dumps({"mode": "linear", "rows": rows, "chained": chained, "k_sweep": sweep, "producer_forms": forms,
                          "cold_weights": cold}))
        return
    blocks = args.blocks
    m = HipPagedKVCacheManager(blocks, ANCHOR + WINDOW + 16, T, H, D, torch.bfloat16, dev,
                               num_special_tokens=N_SPECIAL, scale_frames=ANCHOR, sliding_window=WINDOW,
                               max_total_frames=256, page_size=PAGE, layout="frame_pages")
    g = torch.Generator(device=dev).manual_seed(1)
    n_sets = 4
    qs, ks, vs = ([torch.randn(T, H, D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
                   for _ in range(n_sets)] for _ in range(3))

    if args.constant_kv:
        for t in ks + vs:
            t.fill_(0.5)

    # inputs of the fused producer: qkv projection output, LayerNorm parameters, rotary table
    qkv_in = torch.randn(T, 3 * H * D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    ln = [torch.rand(D, generator=g, device=dev) + 0.5 for _ in range(4)]
    ang = torch.rand(T, D // 2, generator=g, device=dev) * 6.283185
    rope_cs = torch.stack([ang.cos(), ang.sin()], dim=-1).contiguous()
    q_tmp = torch.empty(T, H, D, dtype=torch.bfloat16, device=dev)

    def prepare(block: int) -> None:
        from lingbot_map_amd import _native as N
        import ctypes as C
        vp = lambda t: C.c_void_p(t.data_ptr())
        N.check(N.lib.lbm_qkv_prepare(vp(qkv_in), N.DTYPE_BF16, vp(ln[0]), vp(ln[1]), vp(ln[2]), vp(ln[3]), 1e-5, 1.0,
                                      vp(rope_cs), N.ROPE_INTERLEAVED, vp(q_tmp), None, None, N.DTYPE_BF16, vp(m.kv_caches[block]),
                                      vp(m._append_rows[0]), T, H, D, PAGE, m._stream_handle()))

    # inputs of the fused residual update + LayerNorm (one frame of the 1024-wide trunk)
    res_x = torch.randn(T, H * D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    res_y = torch.randn(T, H * D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    res_p = [torch.rand(H * D, generator=g, device=dev) + 0.5 for _ in range(3)]
    res_o = [torch.empty_like(res_x) for _ in range(2)]

    def residual() -> None:
        from lingbot_map_amd import _native as N
        import ctypes as C
        vp = lambda t: C.c_void_p(t.data_ptr())
        N.check(N.lib.lbm_residual_norm(vp(res_x), vp(res_y), N.DTYPE_BF16, vp(res_p[0]), vp(res_p[1]), vp(res_p[2]), 1e-5,
                                        vp(res_o[0]), vp(res_o[1]), T, H * D, m._stream_handle()))

    def frame(i: int) -> None:
        for b in range(blocks):
            j = (i + b) % n_sets
            # evicted frames leave no trajectory memory here, so the KV set stays at 17,068 tokens
            m.step(b, qs[j], ks[j], vs[j], keyframe=[True], cross_frame_special=False)

    kv_tokens = (ANCHOR + WINDOW) * T
    if args.mode == "attention_frame":
        from lingbot_map_amd import dense_attention
        fn = lambda: dense_attention(qs[0], ks[0], vs[0])
        for _ in range(args.warmup):
            fn()
        ms = kernel_time_ms(fn, 50, torch)
        print(json.dumps({"mode": args.mode, "launches": 200, "avg_launch_us": ms * 1e3,
                          "tflops": 4.0 * T * T * H * D / (ms * 1e-3) * 1e-12}))
        return
    if args.mode == "attention_f32_few":
        # the camera head's shape after 10,000 frames: one fp32 query token, 16 heads of 128
        frames_c = 10000
        mc = HipPagedKVCacheManager(1, frames_c + 16, 1, 16, 128, torch.float32, dev, num_special_tokens=0, scale_frames=8,
                                    sliding_window=frames_c + 8, max_total_frames=frames_c + 16, force_fp32=True,
                                    page_size=PAGE, layout="frame_pages")
        torch.manual_seed(0)
        tok = [torch.randn(1, 16, 128, device=dev) for _ in range(3)]
        for _ in range(frames_c):
            mc.append_frame(0, tok[1], tok[2])
        mc._plan(0, [False])
        fn = lambda: mc._attend_planned(0, tok[0], None, None)
        for _ in range(args.warmup):
            fn()
        ms = event_time_ms(fn, args.steps, torch)
        print(json.dumps({"mode": args.mode, "launches": args.steps, "avg_launch_us": ms * 1e3,
                          "gbps": frames_c * 16 * 128 * 4 * 2 / (ms * 1e-3) * 1e-9}))
        return
    if args.mode == "attention_f32":
        # config 1's last frame: 1004 fp32 queries over 8 cached frames (8032 tokens)
        m32 = HipPagedKVCacheManager(1, 32, T, H, D, torch.float32, dev, num_special_tokens=N_SPECIAL, scale_frames=1,
                                     sliding_window=16, max_total_frames=32, force_fp32=True, page_size=PAGE,
                                     layout="frame_pages")
        torch.manual_seed(0)
        for _ in range(8):
            m32.append_frame(0, torch.randn(T, H, D, device=dev) / 8, torch.randn(T, H, D, device=dev) / 8)
        q32 = torch.randn(T, H, D, device=dev) / 8
        m32._plan(0, [False])
        fn = lambda: m32._attend_planned(0, q32, None, None)
        for _ in range(args.warmup):
            fn()
        ms = event_time_ms(fn, args.steps, torch)
        print(json.dumps({"mode": args.mode, "launches": args.steps, "avg_launch_us": ms * 1e3,
                          "tflops": 4.0 * T * 8 * T * H * D / (ms * 1e-3) * 1e-12}))
        return
    if args.mode != "full":
        # fill the anchor and the window with appends only, so that a profiler sees nothing
        # but --steps + --warmup launches of the one kernel at the steady-state shape
        for i in range(ANCHOR + WINDOW):
            for b in range(2):
                m.append_frame(b, ks[i % n_sets], vs[i % n_sets])
                m.evict_frames(b, ANCHOR, WINDOW, cross_frame_special=False)
        m._plan(0, [False])
        assert m._plan_tokens[0][0] == kv_tokens == 17068
        ops = m._ops([{"ops": 16, "expect_kv_tokens": kv_tokens}])
        fn = {"attention": lambda: m._attend_planned(1, qs[0], None, None),
              "append": lambda: m._scatter(1, m._append_rows[0], ks[0], vs[0]),
              "prepare": lambda: prepare(1),
              "residual": residual,
              "tables": lambda: m._tables_step(0, ops, kv_rows=True)}[args.mode]
        for _ in range(args.warmup):
            fn()
        ms = event_time_ms(fn, args.steps, torch)
        print(json.dumps({"mode": args.mode, "launches": args.steps, "avg_launch_us": ms * 1e3}))
        return
    for i in range(ANCHOR + WINDOW):       # fill the anchor and the window
        frame(i)
    assert m._plan_tokens[0][0] == kv_tokens == 17068
    for i in range(args.warmup):
        frame(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        frame(i)
    torch.cuda.synchronize()
    total = time.perf_counter() - t0
    assert m.device_header()["error"] == 0
    ms_per_step = total / args.steps * 1e3
    fps = args.steps / total

    # the same frame - table step + 24 x (append + attention), keyframes - captured once and replayed
    # as one HIP graph (the device-side tables make every steady-state frame the same launches)
    from lingbot_map_amd import GraphedFrame

    def frame_fn(q, k, v):
        out = None
        for b in range(blocks):
            out = m.step(b, q, k, v, keyframe=None, cross_frame_special=False)
        return out

    graphed = GraphedFrame(m, frame_fn, [qs[0], ks[0], vs[0]], cross_frame_special=False)
    for i in range(args.warmup):
        graphed(qs[i % n_sets], ks[i % n_sets], vs[i % n_sets])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        graphed(qs[i % n_sets], ks[i % n_sets], vs[i % n_sets])
    torch.cuda.synchronize()
    total_graph = time.perf_counter() - t0
    assert m.device_header()["error"] == 0 and m._plan_tokens[0][0] == kv_tokens

    # ---- per-kernel timings with HIP events on the launch stream
    flops = 4.0 * T * kv_tokens * H * D
    m._plan(0, [False])   # the row table of the same visible tokens with every row in the pool (the steps' tables name the newest frame by the caller's rows)
    assert m._plan_tokens[0][0] == kv_tokens
    attn_ms = event_time_ms(lambda: m._attend_planned(1, qs[0], None, None), 500, torch)
    append_ms = kernel_time_ms(lambda: m._scatter(1, m._append_rows[0], ks[0], vs[0]), 100, torch)
    ops = m._ops([{"ops": 16, "expect_kv_tokens": kv_tokens}])
    tables_ms = kernel_time_ms(lambda: m._tables_step(0, ops, kv_rows=True), 100, torch)
    attn_tflops = flops / (attn_ms * 1e-3) * 1e-12
    append_bytes = 2 * 2 * T * H * D * 2
    append_gbps = append_bytes / (append_ms * 1e-3) * 1e-9
    prepare_ms = kernel_time_ms(lambda: prepare(1), 100, torch)
    prepare_bytes = (3 + 3) * T * H * D * 2 + rope_cs.numel() * 4   # read qkv, write q and the K/V rows, read the table
    prepare_gbps = prepare_bytes / (prepare_ms * 1e-3) * 1e-9
    residual_ms = kernel_time_ms(residual, 100, torch)
    residual_bytes = 4 * T * H * D * 2    # read x and y, write x_out and the LayerNorm output
    residual_gbps = residual_bytes / (residual_ms * 1e-3) * 1e-9

    line = {
        "metric": METRIC, "value": fps, "unit": "frames/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"config 2: 518x378 streaming, {T} tokens/frame, page {PAGE}, {ANCHOR} anchor + "
                               f"{WINDOW} window frames = {kv_tokens} KV tokens, {H} heads x {D}, {blocks} global "
                               f"blocks per frame (tables step + per block paged append + paged attention)",
                   "blocks": blocks, "kv_tokens": kv_tokens, "q_tokens": T, "page_size": PAGE},
        "roofline": {"bound": "mfma", "achieved": attn_tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": attn_tflops / PEAK_BF16_TFLOPS, "traffic": ATTN_TRAFFIC_BYTES,
                     "traffic_main_kernel": (ATTN_MAIN_KIB[0] * 2.0 + ATTN_MAIN_KIB[1]) * 1024.0,
                     "algorithmic_bytes": 2.0 * kv_tokens * H * D * 2 + 2.0 * T * H * D * 2,
                     "kernel": "lbm_attn_bf16_d64_kernel + lbm_attn_combine_bf16_kernel (one lbm_attn_run)",
                     "flop_per_launch": flops, "avg_launch_us": attn_ms * 1e3},
        "attention_tflops": attn_tflops,
        "hot_path_hip_graph": {"value": args.steps / total_graph, "unit": "frames/s", "ms_per_step": total_graph / args.steps * 1e3,
                               "what": "the same keyframe step (table step + per block append + attention) replayed as one HIP "
                                       "graph through GraphedFrame; `value` above is the eager loop over the manager's step()"},
        "append": {"bound": "hbm", "achieved": append_gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                   "frac": append_gbps / PEAK_HBM_GBPS, "bytes_per_launch": append_bytes,
                   "avg_launch_us": append_ms * 1e3},
        "qkv_prepare": {"bound": "hbm", "achieved": prepare_gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                        "frac": prepare_gbps / PEAK_HBM_GBPS, "bytes_per_launch": prepare_bytes,
                        "avg_launch_us": prepare_ms * 1e3,
                        "what": "fused q/k LayerNorm + rotary + layout + paged append (replaces the append pass "
                                "when the block feeds the qkv projection output; not in `value`'s timed loop)"},
        "residual_norm": {"bound": "hbm", "achieved": residual_gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                          "frac": residual_gbps / PEAK_HBM_GBPS, "bytes_per_launch": residual_bytes,
                          "avg_launch_us": residual_ms * 1e3,
                          "what": "x + ls(y) fused with the following LayerNorm, 1004 x 1024 bf16 (not in `value`'s timed loop)"},
        "tables_step_us": tables_ms * 1e3,
        "attention_shapes": attention_shapes(torch),
        "hbm_kernels_4_streams": hbm_kernels_4_streams(torch),
        "camera_head_cache": camera_head_cache(torch),
        "config3_stream": config3_stream(torch),
    }
    if not args.no_aggregator:
        del m
        line["aggregator_step"] = aggregator_step(torch, blocks, 20, 3)
        torch.cuda.empty_cache()
        # config 5: four independent streams with windows 4 / 8 / 16 / 16 as one ragged batch
        line["aggregator_step_4_streams"] = aggregator_step(torch, blocks, 10, 2, windows=(4, 8, 16, 16))
        torch.cuda.empty_cache()
        # config 4: keyframe interval 4 - three of four frames only read the cache
        line["aggregator_step_keyframe_interval_4"] = aggregator_step(torch, blocks, 20, 3, keyframe_interval=4)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(torch, kv_tokens, blocks)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
