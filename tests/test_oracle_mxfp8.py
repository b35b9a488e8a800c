"""Pins the oracle of the activation-quantized MXFP8 form against independent numpy closed forms, and
checks the launchers' argument rules (src/kernels/mxfp8_gemm.cu:217-227, :248-250), which run before
anything touches a GPU."""
import ctypes as C

import numpy as np
import pytest

import mxfp8_data as md
import oracle_lib as orc
from np_ref import bf16_bits_to_f64


def oracle_quantize(x, rows, k):
    codes = np.empty((rows, k), dtype=np.uint8)
    scales = np.empty((rows, k // 32), dtype=np.uint8)
    orc.oracle().orc_mxfp8_quantize_rows(orc.p(x), x.shape[1], rows, k, orc.p(codes), orc.p(scales))
    return codes, scales


@pytest.mark.parametrize("maker", [md.all_finite_bf16, md.boundary_rows])
def test_quantizer_matches_closed_form(maker):
    x, rows, k = maker()
    codes, scales = oracle_quantize(x, rows, k)
    want_codes, want_scales = md.quantize_closed_form(x, rows, k)
    assert np.array_equal(scales, want_scales)
    assert np.array_equal(codes, want_codes)


def test_quantizer_known_points():
    # amax 448 -> scale 1; one bf16 step above -> scale 2 and 448 / 2 + rounds; zero group -> byte 0, signed zeros kept.
    x = np.zeros((1, 96), dtype=np.uint16)
    x[0, 0] = md.f32_to_bf16_bits(np.float32(448.0))
    x[0, 1] = md.f32_to_bf16_bits(np.float32(-1.0))
    x[0, 32] = md.f32_to_bf16_bits(np.float32(450.0))
    x[0, 33] = md.f32_to_bf16_bits(np.float32(2.0))
    x[0, 65] = 0x8000
    codes, scales = oracle_quantize(x, 1, 96)
    assert scales.tolist() == [[127, 128, 0]]
    assert codes[0, 0] == 0x7E and codes[0, 1] == 0xB8          # 448, -1.0
    assert codes[0, 32] == 0x76 and codes[0, 33] == 0x38        # 225 -> 224 (ties to even), 1.0
    assert codes[0, 64] == 0x00 and codes[0, 65] == 0x80


def test_swiglu_oai_matches_numpy_and_closed_points():
    rng = np.random.default_rng(5)
    rows, k, stride = 7, 64, 68
    gate = md.f32_to_bf16_bits(rng.normal(0, 6, size=(rows, stride)).astype(np.float32))
    up = md.f32_to_bf16_bits(rng.normal(0, 6, size=(rows, stride)).astype(np.float32))
    gate[0, 0], up[0, 0] = 0x0000, md.f32_to_bf16_bits(np.float32(3.0))      # g = 0 -> 0
    gate[0, 1], up[0, 1] = md.f32_to_bf16_bits(np.float32(2.0)), md.f32_to_bf16_bits(np.float32(-1.0))  # u + 1 = 0
    gate[0, 2], up[0, 2] = md.f32_to_bf16_bits(np.float32(100.0)), md.f32_to_bf16_bits(np.float32(-100.0))
    alpha, limit = np.float32(1.702), np.float32(7.0)
    exact = np.empty((rows, k))
    rounded = np.empty((rows, k), dtype=np.uint16)
    orc.oracle().orc_swiglu_oai(orc.p(gate), orc.p(up), stride, rows, k, alpha, limit, orc.p(exact), orc.p(rounded))
    g = np.minimum(bf16_bits_to_f64(gate[:, :k]), 7.0)
    u = np.clip(bf16_bits_to_f64(up[:, :k]), -7.0, 7.0)
    want = g / (1 + np.exp(-float(alpha) * g)) * (u + 1)
    assert np.allclose(exact, want, rtol=1e-14, atol=0)
    assert exact[0, 0] == 0 and exact[0, 1] == 0
    assert exact[0, 2] == pytest.approx(7.0 / (1 + np.exp(-float(alpha) * 7.0)) * -6.0, rel=1e-14)
    # the rounded form is the nearest bf16 of the exact one
    back = bf16_bits_to_f64(rounded)
    ulp = np.ldexp(1.0, np.floor(np.log2(np.maximum(np.abs(want), 1e-300))).astype(np.int64) - 7)
    assert np.all(np.abs(back - want) <= ulp / 2 + 1e-300)


@pytest.mark.parametrize("m,n,k,seed", [(1, 1, 64, 1), (17, 73, 128, 2), (5, 9, 320, 3)])
def test_gemm_oracle_matches_numpy(m, n, k, seed):
    a, a_s, w, w_s = md.gemm_case(m, n, k, seed)
    out = np.empty((m, n))
    mag = np.empty((m, n))
    orc.oracle().orc_mxfp8_gemm(orc.p(a), orc.p(a_s), orc.p(w), orc.p(w_s), m, n, k, orc.p(out), orc.p(mag))
    ad, wd = md.dequant(a, a_s), md.dequant(w, w_s)
    assert np.allclose(out, ad @ wd.T, rtol=1e-12, atol=1e-12 * np.abs(mag).max())
    assert np.allclose(mag, np.abs(ad) @ np.abs(wd).T, rtol=1e-12)
    if m > 1:
        assert np.all(out[0] == 0)


def test_launchers_reject_what_the_reference_rejects():
    from dgpp_amd import _lib

    lib = _lib.load()
    buf = (C.c_uint8 * 4096)()
    p = C.addressof(buf)
    p = (p + 15) & ~15
    ok, bad = 0, 1      # DGPP_OK, DGPP_INVALID_ARGUMENT

    def gemm(m, n, k, stride=0, tile=0, f32=False):
        fn = lib.dgpp_launch_mxfp8_gemm_f32 if f32 else lib.dgpp_launch_mxfp8_gemm_bf16
        return fn(p, p, p, p, p, m, n, k, None, stride, tile)

    assert gemm(0, 8, 64) == ok and gemm(8, 0, 64) == ok and gemm(-1, 8, 96) == ok     # empty: nothing to check
    for k in (0, -64, 32, 96):
        assert gemm(1, 8, k) == bad
        assert b"multiple of 64" in lib.dgpp_last_error()
    assert gemm(1, 8, 64, stride=7, f32=True) == bad and b"stride" in lib.dgpp_last_error()
    for tile in (1, 4, 24, 128, -8):
        assert gemm(1, 8, 64, tile=tile) == bad and b"output tile" in lib.dgpp_last_error()
    assert lib.dgpp_launch_mxfp8_gemm_bf16(p + 8, p, p, p, p, 1, 8, 64, None, 0, 0) == bad

    def quant(rows, k, stride, fused=False):
        if fused:
            return lib.dgpp_launch_minimax_swiglu_mxfp8_rows(p, p, stride, rows, k, 1.702, 7.0, p, p, None)
        return lib.dgpp_launch_mxfp8_quantize_rows(p, stride, rows, k, p, p, None)

    for fused in (False, True):
        assert quant(0, 48, 1, fused) == ok
        for rows, k, stride in ((1, 0, 32), (1, 48, 48), (1, 64, 32), (1, 32, 34), (70000, 32, 32)):
            assert quant(rows, k, stride, fused) == bad, (rows, k, stride, fused)
    assert lib.dgpp_launch_mxfp8_quantize_rows(p + 4, 32, 1, 32, p, p, None) == bad
    assert lib.dgpp_launch_minimax_swiglu_mxfp8_rows(p, None, 32, 1, 32, 1.702, 7.0, p, p, None) == bad
