"""The built library exports every function include/lbm_paged_attn.h declares, and the
Python binding's constants agree with the header.  No GPU, no compute calls."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lbm_paged_attn.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lbm_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for n in ("lbm_tables_step", "lbm_rows_from_pages", "lbm_kv_append", "lbm_qkv_prepare", "lbm_attn_run",
              "lbm_attn_workspace_bytes", "lbm_tables_words", "lbm_abi_version", "lbm_last_error"):
        assert n in names


def test_library_exports_every_declared_symbol():
    from lingbot_map_amd import _native as N
    lib = C.CDLL(N.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert set(N.SYMBOLS) == set(declared_functions())
    assert N.lib.lbm_abi_version() == N.ABI_VERSION


def test_binding_constants_match_header():
    from lingbot_map_amd import _native as N
    text = open(HEADER).read()
    defs = {m.group(1): int(m.group(2)) for m in re.finditer(r"#define\s+(LBM_[A-Z_0-9]+)\s+(\d+)\b", text)}
    assert defs["LBM_ABI_VERSION"] == N.ABI_VERSION
    assert defs["LBM_MAX_STREAMS"] == N.MAX_STREAMS
    assert defs["LBM_STATIC_SCRATCH_MIB"] == N.STATIC_SCRATCH_MIB
    assert (defs["LBM_OP_RESET"], defs["LBM_OP_ROLLBACK"], defs["LBM_OP_APPEND"], defs["LBM_OP_EVICT"],
            defs["LBM_OP_PLAN"]) == (N.OP_RESET, N.OP_ROLLBACK, N.OP_APPEND, N.OP_EVICT, N.OP_PLAN)
    assert defs["LBM_HDR_WORDS"] == N.HDR_WORDS
    for k, i in N.HDR.items():
        assert defs["LBM_HDR_" + k.upper()] == i
    assert (defs["LBM_DTYPE_BF16"], defs["LBM_DTYPE_F32"]) == (N.DTYPE_BF16, N.DTYPE_F32)
    assert (defs["LBM_LAYOUT_TWO_STREAM"], defs["LBM_LAYOUT_FRAME_PAGES"]) == (N.LAYOUT_TWO_STREAM, N.LAYOUT_FRAME_PAGES)
    # struct sizes: plain int32 fields, no padding
    assert C.sizeof(N.CacheGeom) == 9 * 4 and C.sizeof(N.StepOp) == 8 * 4 and C.sizeof(N.AttnStream) == 5 * 4


def test_host_side_argument_checks_need_no_gpu():
    from lingbot_map_amd import _native as N
    g = N.CacheGeom(0, 7, 3, 4, 1, 19, 21, 0, 40)
    assert N.lib.lbm_tables_words(C.byref(g)) == 16 + 19 + 21 + 1 + 19 + 21 + 0 + 1 + 1
    bad = N.CacheGeom(0, 3, 3, 4, 1, 19, 21, 0, 40)   # no patch tokens
    assert N.lib.lbm_tables_words(C.byref(bad)) == 0
    s = (N.AttnStream * 1)(N.AttnStream(0, 1004, 0, 17068))
    # 4 query tiles x 16 heads x 8 splits = 512 workgroups -> 8 partial results per row
    assert N.lib.lbm_attn_workspace_bytes(s, 1, 16, 64) == 8 * 1004 * 16 * (64 * 2 + 4)
    s1 = (N.AttnStream * 1)(N.AttnStream(0, 9, 0, 64))      # one workgroup per head, nothing to merge
    assert N.lib.lbm_attn_workspace_bytes(s1, 1, 16, 64) == 0
    # at most 8 query rows: partials of the fp32 few-query path, (D + 2) floats per chunk, row and head
    s8 = (N.AttnStream * 1)(N.AttnStream(0, 8, 0, 64))
    assert N.lib.lbm_attn_workspace_bytes(s8, 1, 16, 64) == 1 * 8 * 16 * (64 + 2) * 4
    s9 = (N.AttnStream * 1)(N.AttnStream(0, 1, 0, 10000))
    assert N.lib.lbm_attn_workspace_bytes(s9, 1, 16, 128) == 40 * 1 * 16 * (128 + 2) * 4
    rc = N.lib.lbm_attn_run(None, None, None, None, None, None, s, 1, 16, 64, 16, 0, 0.125, None, 0, None)
    assert rc == N.ERR_INVALID and b"null" in N.lib.lbm_last_error()
    # two streams whose append_rows ranges overlap (an idle stream left at q_begin 0) are refused
    ops = (N.StepOp * 2)(N.StepOp(N.OP_APPEND, 0, 0, 0, 0, 0, 0, 0), N.StepOp(0, 0, 0, 0, 0, 0, 0, 0))
    fake = C.c_void_p(256)   # never dereferenced: the call fails in the argument checks
    rc = N.lib.lbm_tables_step(fake, C.byref(g), 2, ops, fake, None, None, None, None)
    assert rc == N.ERR_INVALID and b"overlap" in N.lib.lbm_last_error()
