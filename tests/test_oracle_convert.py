"""Pins the oracle's scalar conversions: the known answers the reference's own
unit test holds (tests/golden/conversion_kat.json), exhaustive decode against
numpy, and encode against numpy's round-to-nearest-even."""
import json
import os

import numpy as np

import ukref

FLT_MAX = float(np.finfo(np.float32).max)
FLT_MIN = float(np.finfo(np.float32).tiny)


def _val(s):
    neg = s.startswith("-")
    t = s.lstrip("-")
    v = {"FLT_MAX": FLT_MAX, "FLT_MIN": FLT_MIN, "INF": float("inf")}.get(t)
    if v is None:
        v = float(t)
    return -v if neg else v


def _kat():
    with open(os.path.join(os.path.dirname(__file__), "golden", "conversion_kat.json")) as f:
        return json.load(f)


def test_known_answers_of_the_reference_unit_test():
    o = ukref.oracle()
    k = _kat()
    for s, code in k["f32_to_f16"]:
        assert o.oracle_f32_to_f16(_val(s)) == int(code, 16), s
    for s, back in k["f16_round_trip"]:
        for mode in (0, 1):
            assert o.oracle_f16_to_f32(o.oracle_f32_to_f16(_val(s)), mode) == _val(back), s
    for s, code in k["f32_to_bf16"]:
        assert o.oracle_f32_to_bf16(_val(s)) == int(code, 16), s
    for s, back in k["bf16_round_trip"]:
        assert o.oracle_bf16_to_f32(o.oracle_f32_to_bf16(_val(s))) == _val(back), s
    for s, code in k["f32_to_f8e4m3"]:
        # reference flavour (flush) and IEEE flavour agree on every listed input
        assert o.oracle_f32_to_f8e4m3(_val(s), 0, 0) == int(code, 16), s
        assert o.oracle_f32_to_f8e4m3(_val(s), 1, 0) == int(code, 16), s
    for s, back in k["f8e4m3_round_trip"]:
        for ieee in (0, 1):
            assert o.oracle_f8e4m3_to_f32(o.oracle_f32_to_f8e4m3(_val(s), ieee, 0), ieee) == _val(back), s
    nan = o.oracle_f8e4m3_to_f32(o.oracle_f32_to_f8e4m3(float("nan"), 1, 0), 1)
    assert nan != nan
    # denormal input: either flushed or kept is accepted by the reference test
    assert o.oracle_f32_to_f8e4m3(2.0 ** -7, 0, 0) in (0x00, 0x04)
    assert o.oracle_f32_to_f8e4m3(2.0 ** -7, 1, 0) == 0x04
    assert o.oracle_f32_to_f16(2.0 ** -15) in (0x0000, 0x0200)


def test_f16_decode_exhaustive_against_numpy():
    o = ukref.oracle()
    codes = np.arange(65536, dtype=np.uint16)
    want = codes.view(np.float16).astype(np.float32)
    for c in range(65536):
        got = o.oracle_f16_to_f32(c, ukref.F16_IEEE)
        w = want[c]
        assert (np.isnan(w) and got != got) or got == w, hex(c)
        flushed = o.oracle_f16_to_f32(c, ukref.F16_FLUSH)
        if (c & 0x7C00) == 0:  # zero / subnormal codes flush to signed zero
            assert flushed == 0.0 and np.signbit(np.float32(flushed)) == bool(c >> 15)
        elif not np.isnan(w):
            assert flushed == w


def test_f16_encode_against_numpy_in_range():
    o = ukref.oracle()
    rng = np.random.default_rng(0)
    # normal f16 range only: outside it the reference's ukernel helper differs
    # from IEEE on purpose (see narrow16 in oracle.c)
    xs = np.concatenate([
        (rng.standard_normal(20000) * 100).astype(np.float32),
        rng.uniform(2.0 ** -14, 2.0 ** -10, 5000).astype(np.float32),
        rng.uniform(-60000, 60000, 5000).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 2047.5, 2046.5, 65504.0, 65519.99], np.float32)])
    xs = xs[(np.abs(xs) >= 2.0 ** -14) | (xs == 0)]
    want = xs.astype(np.float16).view(np.uint16)
    for x, w in zip(xs, want):
        assert o.oracle_f32_to_f16(float(x)) == int(w), float(x)


def test_bf16_exhaustive_decode_and_rne_encode():
    o = ukref.oracle()
    for c in range(0, 65536, 7):
        got = o.oracle_bf16_to_f32(c)
        want = ukref.bf16_bits_to_f32(np.uint16(c))
        e = (c >> 7) & 0xFF
        if e == 0:
            assert got == 0.0  # subnormals flush (reference common.h:685-686)
        elif np.isnan(want):
            assert got != got
        else:
            assert got == float(want), hex(c)
    rng = np.random.default_rng(1)
    xs = (rng.standard_normal(20000) * 1000).astype(np.float32)
    want = ukref.f32_to_bf16_bits(xs)
    for x, w in zip(xs, want):
        assert o.oracle_f32_to_bf16(float(x)) == int(w)


def test_f8e4m3_all_codes_and_nearest_rounding():
    o = ukref.oracle()
    tab = ukref.f8e4m3_decode_table(ieee=True)
    tab_flush = ukref.f8e4m3_decode_table(ieee=False)
    for c in range(256):
        g = o.oracle_f8e4m3_to_f32(c, 1)
        assert (np.isnan(tab[c]) and g != g) or g == tab[c]
        g = o.oracle_f8e4m3_to_f32(c, 0)
        assert (np.isnan(tab_flush[c]) and g != g) or g == tab_flush[c]
        if not np.isnan(tab[c]):
            assert o.oracle_f32_to_f8e4m3(float(tab[c]), 1, 0) == (c if tab[c] != 0 else (c & 0x80))
    # brute force: the IEEE encoder returns the nearest representable value,
    # ties to the even code; saturation clamps to +-448.
    finite = np.array([c for c in range(128) if not np.isnan(tab[c])])
    vals = tab[finite].astype(np.float64)
    rng = np.random.default_rng(2)
    xs = np.concatenate([rng.uniform(0, 460, 4000), rng.uniform(0, 0.05, 2000),
                         (vals[:-1] + vals[1:]) / 2])  # exact midpoints
    for x in xs:
        code = o.oracle_f32_to_f8e4m3(float(np.float32(x)), 1, 1)
        xf = float(np.float32(x))
        d = np.abs(vals - xf)
        best = d.min()
        cands = finite[d == best]
        if len(cands) == 2:
            want = cands[0] if cands[0] % 2 == 0 else cands[1]
        else:
            want = cands[0]
        assert code == want, (xf, code, want)
    assert o.oracle_f32_to_f8e4m3(1000.0, 1, 1) == 0x7E
    assert o.oracle_f32_to_f8e4m3(-1000.0, 1, 1) == 0xFE
    assert o.oracle_f32_to_f8e4m3(1000.0, 1, 0) == 0x7F
