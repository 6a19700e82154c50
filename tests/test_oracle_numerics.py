"""Pins the oracle's fp16 and e4m3 conversions."""
import json
import os

import numpy as np

import oracle_binding as ob

L = ob.lib()
G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "coopvec_goldens.json")))


def test_f16_decode_exhaustive_against_numpy():
    allh = np.arange(65536, dtype=np.uint16)
    ref = allh.view(np.float16).astype(np.float32)
    got = np.array([L.cvo_f16_to_f32(int(h)) for h in allh], np.float32)
    same = (got == ref) | (np.isnan(got) & np.isnan(ref))
    assert same.all()


def test_f16_rne_against_numpy_including_ties():
    rng = np.random.default_rng(0)
    allh = np.arange(0x7c00, dtype=np.uint16)
    lo = allh[:-1].view(np.float16).astype(np.float64); hi = allh[1:].view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)          # every tie between finite halfs (exact in fp32)
    xs = np.concatenate([
        mid, -mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
        *[rng.standard_normal(5000).astype(np.float32) * s for s in (1e-8, 1e-6, 1e-4, 1, 100, 70000)],
        np.array([65504, 65519.99, 65520, 1e9, np.inf, -np.inf, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -24, 0.0, -0.0],
                 np.float32)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.cvo_f32_to_f16_rne(float(x)) for x in xs], np.uint16)
    assert (got == want).all()


def test_f16_slang_soft_rule():
    # identical to RNE off ties; on ties rounds away from zero; flushes below 2^-24
    rng = np.random.default_rng(1)
    xs = rng.standard_normal(5000).astype(np.float32)
    for x in xs:
        a, b = L.cvo_f32_to_f16_slang(float(x)), L.cvo_f32_to_f16_rne(float(x))
        assert abs(int(a) - int(b)) <= 1
        # it keeps only one guard bit, so it may differ from RNE only when that bit is set
        if a != b:
            assert (np.float32(x).view(np.uint32) >> 12) & 1
    assert L.cvo_f32_to_f16_slang(2049.0) == np.float16(2050).view(np.uint16)
    assert L.cvo_f32_to_f16_rne(2049.0) == np.float16(2048).view(np.uint16)
    assert L.cvo_f32_to_f16_slang(1.0) == 0x3c00 and L.cvo_f32_to_f16_slang(-2.5) == 0xc100
    assert L.cvo_f32_to_f16_slang(2.0 ** -25) == 0 and L.cvo_f32_to_f16_slang(1e6) == 0x7c00
    assert L.cvo_f32_to_f16_slang(2.0 ** -24) == 1
    # the example initialises parameters in [-1,1] with this rule (mlp-training-coopvec.cpp:400-425)
    assert L.cvo_f32_to_f16_slang(0.333251953125) == np.float16(0.333251953125).view(np.uint16)


def test_e4m3_reference_points_and_spec():
    pts = G["e4m3_points"]
    for b, v in pts["decode"].items():
        assert L.cvo_e4m3_to_f32(int(b)) == v
    for v, b in pts["encode"].items():
        assert L.cvo_f32_to_e4m3_sat(float(v)) == b
    # OCP table: bias 7, subnormals m*2^-9, max 448 = 0x7E, 0x7F NaN, no infinities
    vals = np.array([L.cvo_e4m3_to_f32(b) for b in range(256)], np.float32)
    assert vals[0x7e] == 448.0 and np.isnan(vals[0x7f]) and np.isnan(vals[0xff])
    assert vals[1] == 2.0 ** -9 and vals[7] == 7 * 2.0 ** -9 and vals[8] == 2.0 ** -6
    assert (vals[0x80:0xff] == -vals[0x00:0x7f]).all()
    fin = np.sort(vals[:0x7f])
    assert (np.diff(fin) > 0).all()
    # every code round-trips; saturation instead of NaN above the range
    for b in range(256):
        if (b & 0x7f) != 0x7f:
            assert L.cvo_f32_to_e4m3_sat(float(vals[b])) == b
    assert L.cvo_f32_to_e4m3_sat(1e9) == 0x7e and L.cvo_f32_to_e4m3_sat(-500.0) == 0xfe
    assert L.cvo_f32_to_e4m3_sat(float("inf")) == 0x7e and L.cvo_f32_to_e4m3_sat(float("nan")) & 0x7f == 0x7f
    # nearest-even between neighbours: brute force against the value table
    rng = np.random.default_rng(2)
    xs = np.concatenate([rng.standard_normal(4000) * s for s in (0.001, 0.02, 0.5, 10, 300)]).astype(np.float32)
    mids = ((fin[:-1].astype(np.float64) + fin[1:]) / 2).astype(np.float32)
    xs = np.concatenate([xs, mids, np.nextafter(mids, np.float32(1e9)), np.nextafter(mids, np.float32(-1e9))])
    codes = np.arange(0x7f)
    for x in xs:
        a = min(abs(float(x)), 448.0)
        d = np.abs(vals[:0x7f].astype(np.float64) - a)
        best = d.min()
        cands = codes[d == best]
        want = cands[0] if len(cands) == 1 else [c for c in cands if c % 2 == 0][0]
        got = L.cvo_f32_to_e4m3_sat(float(x))
        assert (got & 0x7f) == want, (x, got, want)
        assert (got >> 7) == (1 if np.signbit(x) else 0)
