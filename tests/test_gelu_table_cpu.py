"""The table behind the GEMM's fused GELU epilogue (csrc/gelu_table.inc) against an independent
evaluation: torch's exact-erf GELU in float64 on the CPU, rounded to bf16 through exact integer
arithmetic on the float64 bits.  No GPU."""
import importlib.util
import os
import re

import torch

CSRC = os.path.join(os.path.dirname(__file__), "..", "lingbot-map_amd", "csrc")


def _generator():
    spec = importlib.util.spec_from_file_location("gen_gelu_table", os.path.join(CSRC, "gen_gelu_table.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _committed_entries():
    text = open(os.path.join(CSRC, "gelu_table.inc")).read()
    return [int(x, 16) for x in re.findall(r"0x([0-9a-fA-F]{4})", text)]


def _round_f64_to_bf16_bits(y: torch.Tensor) -> torch.Tensor:
    """Nearest-even rounding of float64 to bf16 by integer arithmetic on the bits: bf16 keeps 7 of
    the 52 fraction bits and has float32's exponent range (all values here are bf16-normal)."""
    b = y.view(torch.int64)
    sign = (b >> 63) & 1
    mag = b & 0x7FFFFFFFFFFFFFFF
    keep = mag >> 45                                   # exponent (11 bits) + 7 fraction bits
    rest = mag & ((1 << 45) - 1)
    half = 1 << 44
    up = (rest > half) | ((rest == half) & ((keep & 1) == 1))
    keep = keep + up.to(torch.int64)                   # a carry into the exponent is the right answer
    e = (keep >> 7) - 1023 + 127                       # re-bias
    assert int(e.min()) > 0 and int(e.max()) < 255
    return (sign << 15) | (e << 7) | (keep & 0x7F)


def test_committed_table_is_the_generators_output():
    gen = _generator()
    entries = _committed_entries()
    assert len(entries) == 2 * gen.HALF == 3840
    assert entries == gen.table()


def test_table_equals_float64_gelu_rounded_once():
    gen = _generator()
    bits = torch.tensor([(neg << 15) | ((gen.E0 << 7) + i) for neg in (0, 1) for i in range(gen.HALF)], dtype=torch.int32)
    v = bits.to(torch.uint16).view(torch.bfloat16).double()
    assert float(v.abs().min()) == 2.0 ** -12 and float(v.abs().max()) < 8.0
    want = _round_f64_to_bf16_bits(torch.nn.functional.gelu(v))
    got = torch.tensor(_committed_entries(), dtype=torch.int64)
    assert torch.equal(got, want)


def test_closed_forms_outside_the_table():
    """Below 2^-12 the epilogue returns v / 2, from 8 up v (positive) or -0 (negative): what
    float32 GELU gives after the rounding to bf16, for every bf16 value out there."""
    bits = torch.arange(65536, dtype=torch.int32)
    exp_field = (bits >> 7) & 0xFF
    mag = bits & 0x7FFF
    finite = exp_field < 0xFE      # (torch's CPU kernel forms 2 v on the way, which overflows in the last binade)
    v = bits.to(torch.uint16).view(torch.bfloat16)
    ref = torch.nn.functional.gelu(v.float()).to(torch.bfloat16)
    small = finite & (mag < ((127 - 12) << 7))
    assert torch.equal((0.5 * v.float()).to(torch.bfloat16)[small].float(), ref[small].float())
    big_pos = finite & (mag >= ((127 + 3) << 7)) & (bits < 0x8000)
    assert torch.equal(v[big_pos], ref[big_pos])
    big_neg = finite & (mag >= ((127 + 3) << 7)) & (bits >= 0x8000)
    assert (ref[big_neg].float() == 0).all()
