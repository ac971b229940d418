"""lbm_attn_run_static: the attention entry point that allocates nothing (its split-KV partials
live in a static device array inside the library) against lbm_attn_run with a caller-owned
workspace.  Same kernels, same schedule: the outputs must agree bit for bit.  Two calls in a
row on the shared array, the second with a smaller batch, then a batch whose partials exceed
the array is refused without a launch."""
import ctypes as C
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def ptr(t):
    return C.c_void_p(t.data_ptr())


def _case(seed, streams_qkv, H, S, dev):
    """Random pool, shuffled row table, one (q_begin, q_rows, kv_row_begin, kv_tokens) per stream."""
    g = torch.Generator().manual_seed(seed)
    D = 64
    n_q = sum(q for q, _ in streams_qkv)
    n_kv = sum(kv for _, kv in streams_qkv)
    pages = -(-(n_kv + 29) // S)
    pool = torch.randn(pages, 2, S, H, D, generator=g).to(torch.bfloat16)
    q = torch.randn(n_q, H, D, generator=g).to(torch.bfloat16)
    perm = torch.randperm(pages * S, generator=g)[:n_kv]
    rows = ((perm // S) * 2 * S + perm % S).to(torch.int32)
    streams, qo, ko = [], 0, 0
    for nq, nk in streams_qkv:
        streams.append((qo, nq, ko, nk, 0))
        qo += nq
        ko += nk
    return q.to(dev), pool.to(dev), rows.to(dev), streams


def test_static_scratch_entry_point_matches_workspace_entry_point():
    from lingbot_map_amd import _native as N
    from oracle.sdpa_cache import sdpa_nhd
    dev = torch.device("cuda:0")
    H, D, S = 16, 64, 16
    # first a launch whose KV axis is split across workgroups (partials in the scratch array),
    # then a smaller one that reuses the front of the array the first call left dirty
    for seed, shape in ((11, [(1004, 9000)]), (12, [(70, 6000), (9, 4500)])):
        q, pool, rows, streams = _case(seed, shape, H, S, dev)
        arr = (N.AttnStream * len(streams))(*[N.AttnStream(*s) for s in streams])
        need = int(N.lib.lbm_attn_workspace_bytes(arr, len(streams), H, D))
        assert need > 0, "the case must use split-KV partials, otherwise the scratch array is not exercised"
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        want = torch.full_like(q, float("nan"))
        got = torch.full_like(q, float("nan"))
        scale = 1.0 / math.sqrt(D)
        N.check(N.lib.lbm_attn_run(ptr(q), ptr(pool), ptr(want), None, None, ptr(rows), arr, len(streams), H, D, S,
                                   N.DTYPE_BF16, scale, ptr(ws), need, None))
        N.check(N.lib.lbm_attn_run_static(ptr(q), ptr(pool), ptr(got), None, None, ptr(rows), arr, len(streams),
                                          H, D, S, N.DTYPE_BF16, scale, None))
        torch.cuda.synchronize()
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, want), (seed, (got.float() - want.float()).abs().max().item())
        # and both are the right answer (bf16 bar: max-abs 2e-2, mean-abs 2e-3 against fp32 SDPA)
        flat_k, flat_v = pool[:, 0].reshape(-1, H, D).cpu(), pool[:, 1].reshape(-1, H, D).cpu()
        slot = lambda r: (r // (2 * S)) * S + r % (2 * S)
        for (qb, nq, kb, nk, _) in streams:
            idx = slot(rows[kb:kb + nk].cpu().long())
            ref = sdpa_nhd(q[qb:qb + nq].cpu(), flat_k[idx], flat_v[idx])
            err = (got[qb:qb + nq].float().cpu() - ref.float()).abs()
            assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    from lingbot_map_amd import _native as N
    torch.zeros(1, device="cuda:0")   # a current device for the library's lookup
    H, D = 64, 64
    big = [(0, 2000, 0, 1000000, 0), (2000, 512, 0, 67068, 0), (2512, 5000, 0, 1000000, 0), (7512, 2000, 0, 1000000, 0)]
    arr = (N.AttnStream * len(big))(*[N.AttnStream(*s) for s in big])
    assert int(N.lib.lbm_attn_workspace_bytes(arr, len(big), H, D)) > (N.STATIC_SCRATCH_MIB << 20)
    rc = N.lib.lbm_attn_run_static(None, None, None, None, None, None, arr, len(big), H, D, 16, N.DTYPE_BF16, 0.125, None)
    assert rc == N.ERR_WORKSPACE
    msg = N.lib.lbm_last_error().decode()
    assert "static" in msg and "lbm_attn_run" in msg
