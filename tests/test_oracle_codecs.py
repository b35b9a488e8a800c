"""Pins the oracle's scalar codecs (and the library's host codecs, which must agree bit for bit):
closed forms over every code, the reference's unit-test known answers
(tests/unit/fp8_test.cpp:29-131, tests/unit/fp4_test.cpp:41-96), and — where oracle/_ref was
built — the compiled reference over every code and a dense float sweep."""
import math
import struct

import numpy as np
import pytest

import oracle_lib as orc
from dgpp_amd import _lib


def f32(x):
    return struct.unpack("<f", struct.pack("<f", x))[0]


def bits_of(x):
    return struct.unpack("<I", struct.pack("<f", x))[0]


def from_bits(u):
    return struct.unpack("<f", struct.pack("<I", u))[0]


@pytest.fixture(scope="module")
def o():
    return orc.oracle()


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def e4m3_closed_form(c):
    s = -1.0 if c & 0x80 else 1.0
    e, m = (c >> 3) & 0xF, c & 7
    if e == 15 and m == 7:
        return math.nan
    if e == 0:
        return s * m * 2.0 ** -9
    return s * (1 + m / 8) * 2.0 ** (e - 7)


def test_e4m3_decode_table_closed_form_and_kats(o, lib):
    for c in range(256):
        want = e4m3_closed_form(c)
        for fn in (o.orc_e4m3_to_f32, lib.dgpp_e4m3_to_f32):
            got = fn(c)
            assert (math.isnan(got) and math.isnan(want)) or got == want, hex(c)
    assert o.orc_e4m3_to_f32(0x38) == 1.0 and o.orc_e4m3_to_f32(0x40) == 2.0 and o.orc_e4m3_to_f32(0x7E) == 448.0
    assert 0 < o.orc_e4m3_to_f32(0x01) < 0.0025
    assert math.copysign(1, lib.dgpp_e4m3_to_f32(0x80)) == -1.0


def test_e4m3_encode_kats_roundtrip_and_half_quantum(o, lib):
    for enc in (o.orc_f32_to_e4m3, lib.dgpp_f32_to_e4m3):
        assert enc(0.0) == 0x00 and enc(-0.0) == 0x80
        assert enc(1000.0) == 0x7E and enc(-1000.0) == 0xFE
        assert enc(448.0) == 0x7E and enc(464.0) == 0x7E and enc(math.inf) == 0x7E
        assert enc(from_bits(0x7FC00001)) == 0x7F and enc(from_bits(0xFFC00001)) == 0xFF
        for c in range(256):
            if (c & 0x7F) == 0x7F:
                continue
            assert enc(e4m3_closed_form(c)) == c, hex(c)
        # ties go to the even code: midway between codes c and c+1
        for c in range(0, 0x7E):
            mid = (e4m3_closed_form(c) + e4m3_closed_form(c + 1)) / 2
            assert f32(mid) == mid
            assert enc(mid) == (c if c % 2 == 0 else c + 1), hex(c)
        # dense sweep: never NaN for finite input, error within half a quantum, saturation exact
        x = 1e-10
        while x <= 500.0:
            for v in (f32(x), -f32(x)):
                code = enc(v)
                assert (code & 0x7F) != 0x7F
                back = e4m3_closed_form(code)
                if abs(v) > 448.0:
                    assert back == math.copysign(448.0, v)
                else:
                    a = abs(back)
                    q = 2.0 ** -9 if a < 2.0 ** -6 else 2.0 ** (math.floor(math.log2(a)) - 3)
                    assert abs(back - v) <= q * 0.5000001 + 1e-12
            x *= 1.003


def test_bf16_codec(o, lib):
    for enc, dec in ((o.orc_f32_to_bf16, o.orc_bf16_to_f32), (lib.dgpp_f32_to_bf16, lib.dgpp_bf16_to_f32)):
        for b in range(0, 65536, 7):
            v = dec(b)
            assert bits_of(v) == b << 16 or math.isnan(v)
            if not math.isnan(v):
                assert enc(v) == b
        # reference KATs: every NaN payload -> canonical quiet NaN with the sign kept
        for u in (0x7FC00000, 0x7FFFFFFF, 0xFFC00001, 0x7F800001, 0xFF800001):
            assert enc(from_bits(u)) == (0xFFC0 if u >> 31 else 0x7FC0)
        assert enc(from_bits(0x7F7FFFFF)) == 0x7F80 and enc(math.inf) == 0x7F80 and enc(-math.inf) == 0xFF80
        # round to nearest even at the tie, both parities
        assert enc(from_bits(0x3F808000)) == 0x3F80 and enc(from_bits(0x3F818000)) == 0x3F82
        assert enc(from_bits(0x3F808001)) == 0x3F81


def test_e2m1_codec(o, lib):
    want = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for enc, dec in ((o.orc_f32_to_e2m1, o.orc_e2m1_to_f32), (lib.dgpp_f32_to_e2m1, lib.dgpp_e2m1_to_f32)):
        for m in range(8):
            assert dec(m) == want[m] and dec(m | 8) == -want[m]
        assert dec(0xF1 & 0xF) == 0.5 and dec(0xF1 >> 4) == -6.0  # low nibble = even element
        for m in range(8):
            assert enc(want[m]) == m and enc(-want[m]) == (m | 8 if m else 8)
        ties = {0.25: 0, 0.75: 2, 1.25: 2, 1.75: 4, 2.5: 4, 3.5: 6, 5.0: 6}
        for v, c in ties.items():
            assert enc(v) == c and enc(-v) == (c | 8)
        assert enc(0.2500001) == 1 and enc(0.7499999) == 1 and enc(5.0000005) == 7
        assert enc(100.0) == 7 and enc(-math.inf) == 15 and enc(math.nan) & 7 == 7


def test_e2m1_times_e4m3_is_exact_in_bf16_for_every_pair(o):
    """tests/unit/fp4_test.cpp:41-61: the lemma the NVFP4 kernels rely on."""
    n = 0
    for code in range(16):
        w = o.orc_e2m1_to_f32(code)
        for sc in range(256):
            s = o.orc_e4m3_to_f32(sc)
            if math.isnan(s):
                continue
            exact = w * s  # python float: exact for these magnitudes
            assert f32(exact) == exact
            assert o.orc_bf16_to_f32(o.orc_f32_to_bf16(exact)) == exact
            n += 1
    assert n == 16 * 254


def test_e8m0_codec(o, lib):
    for dec, ceil in ((o.orc_e8m0_to_f32, o.orc_e8m0_ceil_log2), (lib.dgpp_e8m0_to_f32, lib.dgpp_e8m0_ceil_log2)):
        for b in range(255):
            assert dec(b) == 2.0 ** (b - 127)
        assert math.isnan(dec(255))
        assert bits_of(dec(0)) == 0x00400000
        # ceil(log2 x) for every positive finite bf16 value (tests/cuda/mxfp8_gemm_test.cu:61-119 sweeps the same)
        for hb in range(1, 0x7F80):
            x = from_bits(hb << 16)
            want = max(0, min(254, math.ceil(math.log2(x)) + 127)) if hb >= 0x80 else (1 if hb & 0x7F else 0)
            if hb < 0x80:  # fp32 subnormals: the field rule gives exponent field 0 (+1 with mantissa bits)
                want = 1
            assert ceil(x) == want, hex(hb)
        assert ceil(0.0) == 0 and ceil(1.0) == 127 and ceil(1.0000001) == 128 and ceil(math.inf) == 254


def test_codecs_match_compiled_reference(o, lib):
    r = orc.ref()
    if r is None:
        pytest.skip("oracle/_ref not built (no reference checkout)")
    for c in range(256):
        for a, b, d in ((o.orc_e4m3_to_f32, r.ref_e4m3_to_f32, lib.dgpp_e4m3_to_f32),
                        (o.orc_e8m0_to_f32, r.ref_e8m0_to_f32, lib.dgpp_e8m0_to_f32)):
            x, y, z = a(c), b(c), d(c)
            assert (math.isnan(x) and math.isnan(y) and math.isnan(z)) or (bits_of(x) == bits_of(y) == bits_of(z)), c
    for c in range(16):
        assert bits_of(o.orc_e2m1_to_f32(c)) == bits_of(r.ref_e2m1_to_f32(c)) == bits_of(lib.dgpp_e2m1_to_f32(c))
    rng = np.random.default_rng(11)
    # finite floats across the interesting ranges plus raw random bit patterns (no infinities: the
    # reference's exponent search does not terminate on them)
    vals = np.concatenate([
        rng.normal(0, 1, 30000), rng.normal(0, 200, 20000), rng.normal(0, 0.01, 20000),
        np.exp2(rng.uniform(-30, 12, 30000)) * rng.choice([-1, 1], 30000),
    ]).astype(np.float32)
    raw = rng.integers(0, 2 ** 32, 40000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    raw = raw[np.isfinite(raw) | np.isnan(raw)]
    for v in np.concatenate([vals, raw]).tolist():
        assert o.orc_f32_to_e4m3(v) == r.ref_f32_to_e4m3(v) == lib.dgpp_f32_to_e4m3(v), v
        assert o.orc_f32_to_e2m1(v) == r.ref_f32_to_e2m1(v) == lib.dgpp_f32_to_e2m1(v), v
        assert o.orc_f32_to_bf16(v) == r.ref_f32_to_bf16(v) == lib.dgpp_f32_to_bf16(v), v
        assert o.orc_e8m0_ceil_log2(v) == r.ref_e8m0_ceil_log2(v) == lib.dgpp_e8m0_ceil_log2(v), v
