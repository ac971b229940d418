"""ctypes binding of the C ABI declared in include/lbm_paged_attn.h.

There is no CPU fallback: importing this module without the built library raises."""
from __future__ import annotations

import contextlib
import ctypes as C
import os

from .build import LIB_PATH

OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_WORKSPACE, ERR_HIP = 0, 1, 2, 3, 4
DTYPE_BF16, DTYPE_F32 = 0, 1
LAYOUT_TWO_STREAM, LAYOUT_FRAME_PAGES = 0, 1
ROPE_INTERLEAVED, ROPE_HALF_SPLIT = 0, 1
LINEAR_BIAS, LINEAR_BIAS_GELU, LINEAR_BIAS_RESIDUAL = 0, 1, 2
MAX_STREAMS = 16
STATIC_SCRATCH_MIB = 64
OP_RESET, OP_ROLLBACK, OP_APPEND, OP_EVICT, OP_PLAN, OP_PLAN_NEWEST_SELF = 1, 2, 4, 8, 16, 32
TERR_NAMES = {1: "patch page pool exhausted", 2: "special page pool exhausted", 4: "window ring full",
              8: "trajectory memory full", 16: "rollback underflow", 32: "visible token count mismatch"}
HDR = {"frame_count": 0, "n_anchor": 1, "win_head": 2, "win_count": 3, "n_free_patch": 4,
       "n_free_special": 5, "n_special_pages": 6, "special_tokens": 7, "n_memory": 8,
       "n_memory_pages": 9, "error": 10, "plan_kv_tokens": 11, "plan_n_pages": 12}
HDR_WORDS = 16
ABI_VERSION = 9


# Scratch memory that the package keeps per device (the K-split workspace of the GEMM, the
# workspace of the cache-less attention) serves one chain of launches at a time.  Code that runs a
# second chain which may overlap the first on the same GPU (another branch of a HIP graph) runs it
# under ``scratch_lane(1)``: every lane has scratch areas of its own.
_scratch_lane = 0


def current_scratch_lane() -> int:
    return _scratch_lane


@contextlib.contextmanager
def scratch_lane(lane: int):
    global _scratch_lane
    before, _scratch_lane = _scratch_lane, int(lane)
    try:
        yield
    finally:
        _scratch_lane = before


class CacheGeom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "layout", "tokens_per_frame", "num_special_tokens", "page_size", "scale_frames",
        "patch_pages", "special_pages", "memory_frames", "pages_per_stream")]


class StepOp(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "ops", "sliding_window", "keep_tokens", "self_tokens", "q_begin", "kv_row_begin",
        "expect_kv_tokens", "page_out_begin")]


class AttnStream(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("q_begin", "q_rows", "kv_row_begin", "kv_tokens", "live_at")]


class RowNorm(C.Structure):
    """``lbm_row_norm``: a LayerNorm folded into the launch that consumes its output."""
    _fields_ = [("stats", C.c_void_p), ("w_colsum", C.c_void_p), ("stats_tiles", C.c_int32), ("eps", C.c_float)]


SYMBOLS = ("lbm_abi_version", "lbm_last_error", "lbm_tables_words", "lbm_tables_step",
           "lbm_rows_from_pages", "lbm_kv_append", "lbm_qkv_prepare", "lbm_residual_norm", "lbm_linear", "lbm_linear_norm", "lbm_linear_stats_tiles", "lbm_linear_workspace_bytes", "lbm_linear_prefetch_hint", "lbm_qkv_linear_prepare", "lbm_qkv_linear_prepare_norm", "lbm_attn_workspace_bytes", "lbm_attn_run", "lbm_attn_run_append", "lbm_attn_run_live",
           "lbm_attn_run_static")


def _load():
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"HIP library {LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(there is no CPU fallback for this path)")
    lib = C.CDLL(LIB_PATH)
    p, i32, vp = C.POINTER, C.c_int32, C.c_void_p
    lib.lbm_abi_version.restype = C.c_int
    lib.lbm_last_error.restype = C.c_char_p
    lib.lbm_tables_words.restype = C.c_int64
    lib.lbm_tables_words.argtypes = [p(CacheGeom)]
    lib.lbm_tables_step.restype = C.c_int
    lib.lbm_tables_step.argtypes = [vp, p(CacheGeom), i32, p(StepOp), vp, vp, vp, vp, vp]
    lib.lbm_rows_from_pages.restype = C.c_int
    lib.lbm_rows_from_pages.argtypes = [vp, vp, p(i32), p(i32), p(i32), i32, i32, vp, vp]
    lib.lbm_kv_append.restype = C.c_int
    lib.lbm_kv_append.argtypes = [vp, vp, i32, vp, i32, vp, i32, i32, i32, i32, vp]
    lib.lbm_qkv_prepare.restype = C.c_int
    lib.lbm_qkv_prepare.argtypes = [vp, i32, vp, vp, vp, vp, C.c_float, C.c_float, vp, i32, vp, vp, vp, i32, vp, vp, i32, i32, i32, i32, vp]
    lib.lbm_residual_norm.restype = C.c_int
    lib.lbm_residual_norm.argtypes = [vp, vp, i32, vp, vp, vp, C.c_float, vp, vp, i32, i32, vp]
    lib.lbm_linear.restype = C.c_int
    lib.lbm_linear.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]
    lib.lbm_linear_norm.restype = C.c_int
    lib.lbm_linear_norm.argtypes = [vp, p(RowNorm), vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp, C.c_size_t, vp]
    lib.lbm_linear_workspace_bytes.restype = C.c_size_t
    lib.lbm_linear_workspace_bytes.argtypes = [i32, i32, i32, i32]
    lib.lbm_linear_prefetch_hint.restype = C.c_int
    lib.lbm_linear_prefetch_hint.argtypes = [vp, C.c_size_t]
    lib.lbm_linear_stats_tiles.restype = i32
    lib.lbm_linear_stats_tiles.argtypes = [i32, i32]
    lib.lbm_qkv_linear_prepare_norm.restype = C.c_int
    lib.lbm_qkv_linear_prepare_norm.argtypes = [vp, p(RowNorm), vp, vp, i32, i32, vp, vp, vp, vp, C.c_float, C.c_float, vp, i32, vp, vp, vp, vp, vp, i32, i32, i32, vp]
    lib.lbm_qkv_linear_prepare.restype = C.c_int
    lib.lbm_qkv_linear_prepare.argtypes = [vp, vp, vp, i32, i32, vp, vp, vp, vp, C.c_float, C.c_float, vp, i32, vp, vp, vp, vp, vp, i32, i32, i32, vp]
    lib.lbm_attn_workspace_bytes.restype = C.c_size_t
    lib.lbm_attn_workspace_bytes.argtypes = [p(AttnStream), i32, i32, i32]
    lib.lbm_attn_run.restype = C.c_int
    lib.lbm_attn_run.argtypes = [vp, vp, vp, vp, vp, vp, p(AttnStream), i32, i32, i32, i32, i32,
                                 C.c_float, vp, C.c_size_t, vp]
    lib.lbm_attn_run_append.restype = C.c_int
    lib.lbm_attn_run_append.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32, p(AttnStream), i32, i32, i32, i32, i32,
                                        C.c_float, vp, C.c_size_t, vp]
    lib.lbm_attn_run_live.restype = C.c_int
    lib.lbm_attn_run_live.argtypes = [vp, vp, vp, vp, vp, vp, vp, p(AttnStream), i32, i32, i32, i32, i32,
                                      C.c_float, vp, C.c_size_t, vp]
    lib.lbm_attn_run_static.restype = C.c_int
    lib.lbm_attn_run_static.argtypes = [vp, vp, vp, vp, vp, vp, p(AttnStream), i32, i32, i32, i32, i32, C.c_float, vp]
    if lib.lbm_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH}: ABI version {lib.lbm_abi_version()}, binding expects {ABI_VERSION}")
    return lib


lib = _load()


class LbmError(RuntimeError):
    pass


def check(rc: int) -> None:
    if rc != OK:
        msg = lib.lbm_last_error().decode("utf-8", "replace")
        if rc == ERR_INVALID:
            raise ValueError(msg)
        raise LbmError(f"lbm error {rc}: {msg}")


def q_scale_log2(sm_scale: float) -> float:
    """The ``q_scale`` to hand the producers so that ``lbm_attn_run`` can be called with
    ``sm_scale = 0``: the softmax scale times log2(e), as a float32 value."""
    import struct
    return struct.unpack("f", struct.pack("f", sm_scale * 1.4426950408889634))[0]


def stream_ptr(device) -> C.c_void_p:
    """The current HIP stream of ``device`` as the ``void*`` the entry points take.  One C call
    instead of building a ``torch.cuda.Stream`` object per launch (5 us each, several hundred per
    aggregator frame)."""
    import torch
    idx = device.index if getattr(device, "index", None) is not None else torch.cuda.current_device()
    return C.c_void_p(torch._C._cuda_getCurrentRawStream(idx))
