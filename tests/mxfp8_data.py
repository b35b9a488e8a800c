"""Inputs and independent numpy closed forms for the activation-quantized MXFP8 form.

The input recipes follow the reference's own kernel test (tests/cuda/mxfp8_gemm_test.cu:96-123 for the
quantizer, :196-208 for the GEMM); the closed forms are evaluated in float64 from the formats' value
tables, sharing no code with the oracle or the library."""
import numpy as np

from np_ref import E4M3, bf16_bits_to_f64

_POS = E4M3[:0x7F]          # codes 0 .. 0x7E ascending: 0 .. 448
NAN_BITS = 0x7FC0


def f32_to_bf16_bits(x):
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def all_finite_bf16(stride=36):
    """Every finite BF16 pattern, signed zeros and subnormals included, as 2040 rows of one 32-group;
    the padding between rows is NaN, which a correct kernel never reads into a group."""
    rows, k = 2040, 32
    x = np.full((rows, stride), NAN_BITS, dtype=np.uint16)
    idx = np.arange(rows * k)
    x[:, :k] = np.where(idx < 32640, idx, (idx - 32640) | 0x8000).astype(np.uint16).reshape(rows, k)
    return x, rows, k


def boundary_rows(pad=4):
    """193 groups per row (a partly filled last block of lanes); each group's largest magnitude is
    446, 448 or 450 times a power of two: just under, on and just over the step of the scale."""
    wide = 6176
    x = np.full((3, wide + pad), NAN_BITS, dtype=np.uint16)
    col = np.arange(wide)
    for row, lead in enumerate((446.0, 448.0, 450.0)):
        maximum = np.ldexp(np.float32(lead), (col // 32) % 49 - 24).astype(np.float32)
        value = np.where(col % 32 == 0, maximum, maximum * ((col % 17 - 8).astype(np.float32)) / np.float32(16))
        x[row, :wide] = f32_to_bf16_bits(value.astype(np.float32))
    return x, 3, wide


def e4m3_rne(v):
    """float64 values (any sign) -> E4M3 codes: nearest, ties to the even code, saturating at 448."""
    mag = np.abs(v)
    hi = np.clip(np.searchsorted(_POS, mag, side="left"), 0, len(_POS) - 1)
    lo = np.clip(hi - 1, 0, None)
    d_lo, d_hi = mag - _POS[lo], _POS[hi] - mag
    pick = np.where(d_hi < d_lo, hi, np.where(d_lo < d_hi, lo, np.where(hi % 2 == 0, hi, lo)))
    pick = np.where(mag >= 448.0, 0x7E, pick)
    return (pick | np.where(np.signbit(v), 0x80, 0)).astype(np.uint8)


def quantize_closed_form(x_bits, rows, k):
    """codes, scales by the rule the reference's test states: exponent = max(-127, ceil(log2(amax / 448)))."""
    v = bf16_bits_to_f64(x_bits[:, :k]).reshape(rows, k // 32, 32)
    amax = np.abs(v).max(axis=2)
    with np.errstate(divide="ignore"):
        exponent = np.where(amax == 0, -127, np.maximum(-127, np.ceil(np.log2(amax / 448.0)))).astype(np.int64)
    codes = e4m3_rne(v * np.ldexp(1.0, -exponent)[:, :, None]).reshape(rows, k)
    return codes, (exponent + 127).astype(np.uint8)


def dequant(codes, scales):
    """E4M3 codes [r, k] with e8m0 scales [r, k / 32] as float64."""
    return E4M3[codes] * np.repeat(np.ldexp(1.0, scales.astype(np.int64) - 127), 32, axis=1)


def gemm_case(m, n, k, seed):
    """Random codes without the NaN pattern, scales 2^-10 .. 2^6 distinct per row and group; with more
    than one row, row 0 of A alternates +0 and -0."""
    rng = np.random.default_rng(seed)

    def codes(r):
        c = rng.integers(0, 256, size=(r, k), dtype=np.uint8)
        return np.where((c & 127) == 127, c & 0xF0, c).astype(np.uint8)

    a, w = codes(m), codes(n)
    a_s = (117 + rng.integers(0, 17, size=(m, k // 32))).astype(np.uint8)
    w_s = (117 + rng.integers(0, 17, size=(n, k // 32))).astype(np.uint8)
    if m > 1:
        a[0] = np.where(np.arange(k) & 1, 128, 0).astype(np.uint8)
    return a, a_s, w, w_s
