"""The library's host encoders (the published weight recipes) against the reference's own encoder
bytes (golden fixture, and live where oracle/_ref exists) and the reference's unit-test KATs
(tests/unit/nvfp4_quant_test.cpp:31-90)."""
from pathlib import Path

import numpy as np
import pytest

import np_ref
import oracle_lib as orc
from dgpp_amd import hostgen as hg

GOLDEN = Path(__file__).resolve().parent / "golden" / "quantizers.npz"


def test_encoders_match_reference_bytes():
    z = np.load(GOLDEN)
    payload, scales, ws2 = hg.encode_nvfp4(z["w"], threads=3)
    assert np.float32(ws2) == z["ws2"]
    assert np.array_equal(payload, z["nvfp4_payload"]) and np.array_equal(scales, z["nvfp4_scales"])
    p8, s8 = hg.encode_fp8_blocks(z["wb"], 128, 128, threads=2)
    assert np.array_equal(p8, z["fp8_payload"]) and np.array_equal(s8, z["fp8_scales"])


def test_encoders_match_live_reference():
    r = orc.ref()
    if r is None:
        pytest.skip("oracle/_ref not built (no reference checkout)")
    for seed in (1, 2, 3):
        w = hg.normal_f32(seed, (5, 64), 0.02 * seed)
        payload, scales, ws2 = hg.encode_nvfp4(w)
        assert np.float32(ws2) == np.float32(r.ref_nvfp4_tensor_scale(float(np.abs(w).max())))
        for i in range(5):
            rp, rs = np.empty(32, np.uint8), np.empty(4, np.uint8)
            row = np.ascontiguousarray(w[i])
            r.ref_nvfp4_encode_row(orc.p(row), 64, ws2, orc.p(rp), orc.p(rs))
            assert np.array_equal(rp, payload[i]) and np.array_equal(rs, scales[i])


def test_nvfp4_kats():
    grid = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], np.float32)
    w = (np.where(np.arange(16) % 2, -1.0, 1.0) * grid[np.arange(16) % 8] * 2.0).astype(np.float32)[None, :]
    payload, scales, ws2 = hg.encode_nvfp4(w)
    assert np.float32(ws2) == np.float32(12.0) / np.float32(2688.0)
    assert scales[0, 0] == 0x7E                              # e4m3(448) exactly
    back = np_ref.dequant_fp4(payload, scales, 16)[0] * ws2
    assert np.allclose(back, w[0], atol=1e-5 * 12)
    payload, scales, ws2 = hg.encode_nvfp4(np.zeros((2, 32), np.float32))
    assert ws2 == 1.0 and not payload.any() and not scales.any()
    # round trip within the format error: 0.2 * block max
    w = hg.normal_f32(5, (7, 96), 0.05)
    w[0, 5] = 0.9
    payload, scales, ws2 = hg.encode_nvfp4(w)
    assert not np.any((scales & 0x7F) == 0x7F)
    back = np_ref.dequant_fp4(payload, scales, 16) * ws2
    bmax = np.abs(w).reshape(7, 6, 16).max(axis=2).repeat(16, axis=1)
    assert np.all(np.abs(back - w) <= 0.2 * bmax + 1e-6)
    assert abs(back[0, 5] - 0.9) < 0.9 * 0.03


@pytest.mark.parametrize("fmt", ["mxfp4", "mxfp8"])
def test_mx_encoders(fmt):
    w = hg.normal_f32(8, (6, 128), 0.02)
    w[2, 32:64] = 0
    w[3, 0] = 6.0 * 2.0 ** -5 if fmt == "mxfp4" else 448.0 * 2.0 ** -5      # amax exactly fmt_max * 2^-5
    fmt_max = 6.0 if fmt == "mxfp4" else 448.0
    payload, scales = (hg.encode_mxfp4 if fmt == "mxfp4" else hg.encode_mxfp8)(w)
    assert scales[2, 1] == 0 and not payload[2, (16 if fmt == "mxfp4" else 32):(32 if fmt == "mxfp4" else 64)].any()
    amax = np.abs(w).reshape(6, 4, 32).max(axis=2)
    nz = amax > 0
    want = np.ceil(np.log2(amax[nz].astype(np.float64) / fmt_max)) + 127    # the ceil-pow2 rule
    got = scales[nz].astype(np.float64)
    assert np.all(np.abs(got - want) <= 1) and np.mean(got == want) > 0.9   # fp32 division may round at a boundary
    assert scales[3, 0] == 127 - 5
    back = np_ref.dequant_fp4(payload, scales, 32) if fmt == "mxfp4" else np_ref.dequant_fp8(payload, scales, 0, 5, False, True)
    s = np.exp2(scales.astype(np.float64) - 127).repeat(32, axis=1)
    step = (1.0 if fmt == "mxfp4" else 16.0) * s          # half the widest grid step of the format
    assert np.all(np.abs(back - w) <= step + 1e-30)       # never saturated: |w| <= fmt_max * scale


def test_generators_are_thread_invariant_and_normal():
    a = hg.normal_f32(42, (3, 5000), 0.02, threads=1)
    b = hg.normal_f32(42, (3, 5000), 0.02, threads=7)
    assert np.array_equal(a, b)
    assert abs(a.std() - 0.02) < 5e-4 and abs(a.mean()) < 5e-4
    assert not np.array_equal(a, hg.normal_f32(43, (3, 5000), 0.02))
    x = hg.normal_bf16(1, (4, 256))
    assert np.array_equal(x, hg.f32_to_bf16(hg.normal_f32(1, (4, 256))))
    ids = hg.zipf_routes(3, 1.1, 32, 8, 128)
    assert ids.shape == (32, 8) and np.all(np.diff(ids, axis=1) > 0) and ids.min() >= 0 and ids.max() < 128
    assert np.bincount(ids.ravel(), minlength=128)[:8].sum() > np.bincount(ids.ravel(), minlength=128)[64:].sum()
