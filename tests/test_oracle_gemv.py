"""The oracle's dequantisation and GEMV against an independent numpy brute force on small shapes,
plus invariants a dropped term / wrong index / transposed operand would break."""
import numpy as np
import pytest

import np_ref
import oracle_lib as orc
from dgpp_amd import hostgen as hg


def close(a, b, tol=1e-12):
    both_nan = np.isnan(a) & np.isnan(b)
    scale = np.maximum(np.abs(b), 1e-30)
    return np.all(both_nan | (np.abs(a - b) <= tol * scale) | ((a == b)))


@pytest.mark.parametrize("group", [16, 32])
def test_fp4_dequant_and_gemv_vs_numpy(group):
    rng = np.random.default_rng(group)
    n, k, m = 37, 192, 3
    payload = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    scales = rng.integers(0, 255, (n, k // group), dtype=np.uint8)
    if group == 16:
        scales[scales == 0x7F] = 0x3A
        scales[2, 3] = 0x7F   # one NaN scale
    else:
        scales = rng.integers(110, 135, (n, k // group), dtype=np.uint8)
        scales[4, 1] = 255
    w = np.empty((n, k), np.float64)
    orc.oracle().orc_dequant_fp4(orc.p(payload), orc.p(scales), group, n, k, orc.p(w))
    want = np_ref.dequant_fp4(payload, scales, group)
    assert np.array_equal(np.isnan(w), np.isnan(want))
    assert np.array_equal(np.nan_to_num(w), np.nan_to_num(want))   # exact: small products of short mantissas
    act = hg.normal_bf16(5, (m, k))
    got = orc.gemv_fp4(act, payload, scales, 3.5, group, m, n, k)
    assert close(got, np_ref.gemv(act, want, 3.5))
    # element (r, c) is picked out by a one-hot activation: pins nibble order and scale indexing
    onehot = np.zeros((1, k), np.uint16)
    for c in (0, 1, 17, 33, k - 1):
        onehot[:] = 0
        onehot[0, c] = 0x3F80
        col = orc.gemv_fp4(onehot, payload, scales, 1.0, group, 1, n, k)[0]
        ok = ~np.isnan(want).any(axis=1)  # a NaN anywhere in a row poisons its dot
        assert np.array_equal(col[ok], want[ok, c])


@pytest.mark.parametrize("rs,cs,e8m0", [(7, 7, False), (5, 5, False), (0, 5, False), (0, 5, True), (6, 4, False)])
def test_fp8_dequant_and_gemv_vs_numpy(rs, cs, e8m0):
    rng = np.random.default_rng(rs * 16 + cs)
    n, k, m = 150, 272, 2
    payload = rng.integers(0, 256, (n, k), dtype=np.uint8)
    payload[payload == 0x7F] = 0x11
    payload[payload == 0xFF] = 0x91
    srows, scols = (n + (1 << rs) - 1) >> rs, (k + (1 << cs) - 1) >> cs
    if e8m0:
        scales = rng.integers(100, 140, (srows, scols), dtype=np.uint8)
        scales[0, 0] = 0
    else:
        scales = np.exp2(rng.uniform(-12, 2, (srows, scols))).astype(np.float32)
    for strict in (True, False):
        w = np.empty((n, k), np.float64)
        orc.oracle().orc_dequant_fp8(orc.p(payload), None if e8m0 else orc.p(scales), orc.p(scales) if e8m0 else None,
                                     n, k, rs, cs, int(strict), orc.p(w))
        want = np_ref.dequant_fp8(payload, scales, rs, cs, strict, e8m0)
        assert np.array_equal(w, want), (rs, cs, strict)
        act = hg.normal_bf16(9, (m, k))
        got = orc.gemv_fp8(act, payload, scales, m, n, k, rs, cs, strict, e8m0)
        assert close(got, np_ref.gemv(act, want))


def test_gemv_linearity_and_zero_k():
    rng = np.random.default_rng(1)
    n, k = 20, 64
    w = hg.normal_f32(3, (n, k), 0.02)
    payload, scales = hg.encode_mxfp4(w)
    a = hg.normal_bf16(4, (1, k))
    two = hg.f32_to_bf16(hg.bf16_to_f32(a) * 2)   # exact doubling in bf16
    r1 = orc.gemv_fp4(a, payload, scales, 1.0, 32, 1, n, k)
    r2 = orc.gemv_fp4(two, payload, scales, 1.0, 32, 1, n, k)
    assert np.array_equal(r2, 2 * r1)
    assert np.array_equal(orc.gemv_fp4(a, payload, scales, 4.0, 32, 1, n, k), r1 / 4.0)
    out = orc.gemv_fp8(np.zeros((2, 0), np.uint16), np.zeros((5, 0), np.uint8), np.ones((1, 1), np.float32), 2, 5, 0)
    assert not out.any()


def test_comparator_semantics():
    """tests/cuda/scale_gemm_test_helpers.hpp:72-100: both the ulp budget and the floor must be exceeded."""
    oracle = np.array([1.0, 100.0, 1e-6, np.nan], dtype=np.float64)
    got = hg.f32_to_bf16(np.array([1.0 + 3 * 2.0 ** -7, 100.0, 5e-4, np.nan], dtype=np.float32))
    rep = orc.compare_bf16(got, oracle, 2.0, 1e-3)
    assert rep.mismatches == 0 and rep.nan_pattern_errors == 0   # 3 ulps at 1.0 is below the 0.1 floor
    rep = orc.compare_bf16(got, oracle, 2.0, 1e-5)
    assert rep.mismatches == 1
    got2 = hg.f32_to_bf16(np.array([1.0, 100.0, 1e-6, 1.0], dtype=np.float32))
    rep = orc.compare_bf16(got2, oracle, 2.0, 1e-3)
    assert rep.nan_pattern_errors == 1 and rep.mismatches == 1
