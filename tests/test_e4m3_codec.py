"""fp8 / fp16 codecs of the oracle, pinned without the reference:
closed-form decode of all 256 codes, round-to-nearest-even on every midpoint between adjacent codes, recorded
known answers, and the CPU library cast of torch (which differs only above the finite range: torch overflows to NaN,
the pipeline saturates).  Two independent encoders (C bit-level, numpy table search) must agree everywhere.
"""
import numpy as np
import pytest
import torch

from oracle import fa8_oracle as fo
from oracle import np_restatement as nr

L = fo.lib()


def closed_form_e4m3(c):
    s, e, m = c >> 7, (c >> 3) & 15, c & 7
    if e == 15 and m == 7:
        return float("nan")
    v = m * 2.0 ** -9 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
    return -v if s else v


def closed_form_e5m2(c):
    s, e, m = c >> 7, (c >> 2) & 31, c & 3
    if e == 31:
        return float("nan") if m else (float("-inf") if s else float("inf"))
    v = m * 2.0 ** -16 if e == 0 else (1 + m / 4) * 2.0 ** (e - 15)
    return -v if s else v


def test_decode_all_codes_closed_form_and_torch():
    t4 = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    t5 = torch.arange(256, dtype=torch.uint8).view(torch.float8_e5m2).float().numpy()
    for c in range(256):
        for got, want, lib_val in ((L.fa8o_e4m3_to_f32(c), closed_form_e4m3(c), t4[c]),
                                   (L.fa8o_e5m2_to_f32(c), closed_form_e5m2(c), t5[c])):
            if np.isnan(want):
                assert np.isnan(got) and np.isnan(lib_val)
            else:
                assert got == want == lib_val
    assert np.array_equal(nr.E4M3_TABLE, np.array([closed_form_e4m3(c) for c in range(256)]), equal_nan=True)
    assert np.array_equal(nr.E5M2_TABLE, np.array([closed_form_e5m2(c) for c in range(256)]), equal_nan=True)


def test_e4m3_facts():
    assert L.fa8o_e4m3_to_f32(0x7E) == 448.0 and L.fa8o_e4m3_to_f32(0x01) == 2.0 ** -9
    assert L.fa8o_e4m3_to_f32(0x08) == 2.0 ** -6 and L.fa8o_e4m3_to_f32(0x38) == 1.0
    finite = [closed_form_e4m3(c) for c in range(256) if not np.isnan(closed_form_e4m3(c))]
    assert len(finite) == 254
    # every finite e4m3 value is exact in fp16
    assert all(float(np.float16(v)) == v for v in finite)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_encode_round_trip_and_midpoints(fmt):
    enc = L.fa8o_f32_to_e4m3 if fmt == "e4m3" else L.fa8o_f32_to_e5m2
    table = nr.E4M3_TABLE if fmt == "e4m3" else nr.E5M2_TABLE
    codes = [c for c in range(128) if np.isfinite(table[c])]
    for c in codes:  # exact values round-trip, both signs
        assert enc(float(table[c])) == c
        assert enc(-float(table[c])) == (c | 0x80)
    for lo, hi in zip(codes[:-1], codes[1:]):
        mid = (table[lo] + table[hi]) / 2  # exactly representable in fp32
        even = lo if lo % 2 == 0 else hi
        assert enc(float(mid)) == even, (lo, hi)
        assert enc(float(np.nextafter(np.float32(mid), np.float32(np.inf)))) == hi
        assert enc(float(np.nextafter(np.float32(mid), np.float32(-np.inf)))) == lo
        assert nr.encode_rne_sat(np.array([mid]), fmt)[0] == even


def test_encode_known_answers_e4m3():
    kat = {0.96875: 0x38, 0.9687399: 0x37, 0.53125: 0x30, 0.59375: 0x32, 0.1: 0x1D, 2.0 ** -10: 0x00,
           2.0 ** -10 * 1.0001: 0x01, 3 * 2.0 ** -10: 0x02, 2.0 ** -11: 0x00, 2.0 ** -6 - 2.0 ** -10: 0x08,
           448.0: 0x7E, 449.0: 0x7E, 464.0: 0x7E, 465.0: 0x7E, 1e9: 0x7E, float("inf"): 0x7E, 0.0: 0x00}
    for x, code in kat.items():
        assert L.fa8o_f32_to_e4m3(x) == code, x
        assert nr.encode_rne_sat(np.array([x]))[0] == code, x
    assert L.fa8o_f32_to_e4m3(-0.0) == 0x80
    assert L.fa8o_f32_to_e4m3(float("nan")) & 0x7F == 0x7F


def test_encode_matches_torch_library_cast_in_range():
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(20000) * s for s in (1e-3, 0.05, 1.0, 30.0)]).astype(np.float32)
    x = np.clip(x, -448, 448)
    want4 = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    want5 = torch.from_numpy(x).to(torch.float8_e5m2).view(torch.uint8).numpy()
    got4 = np.array([L.fa8o_f32_to_e4m3(float(v)) for v in x], dtype=np.uint8)
    got5 = np.array([L.fa8o_f32_to_e5m2(float(v)) for v in x], dtype=np.uint8)
    assert np.array_equal(got4, want4)
    assert np.array_equal(got5, want5)
    assert np.array_equal(nr.encode_rne_sat(x, "e4m3"), want4)
    assert np.array_equal(nr.encode_rne_sat(x, "e5m2"), want5)


def test_fp16_conversion_matches_numpy():
    rng = np.random.default_rng(6)
    x = np.concatenate([rng.standard_normal(20000) * s for s in (1e-7, 1e-4, 1.0, 1000.0, 60000.0)]).astype(np.float32)
    x = np.concatenate([x, np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e10, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25],
                                    dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([L.fa8o_f32_to_f16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)
    for c in range(0, 65536, 7):
        w = np.array([c], dtype=np.uint16).view(np.float16).astype(np.float32)[0]
        g = L.fa8o_f16_to_f32(c)
        assert (np.isnan(w) and np.isnan(g)) or w == g
