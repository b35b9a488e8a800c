"""Pins the oracle of the activation-quantized NVFP4 (W4A4) form: the row quantizer against the reference test's
known-answer rows, closed-form points and an independent numpy float32 restatement of the recipe; the fp64 GEMM of
quantized operands against numpy brute force; and the launchers' argument rules (src/kernels/moe_w4a4.cu:598-634,
:641-646), which run before anything touches a GPU."""
import numpy as np
import pytest

import nvfp4_data as nd
import oracle_lib as orc
from np_ref import bf16_bits_to_f64


def oracle_quantize(x, rows, k, static_gs=0.0):
    ss = nd.scale_stride(k)
    codes = np.empty((rows, k // 2), np.uint8)
    scales = np.full((rows, ss), 0xAA, np.uint8)
    gs = np.empty(rows, np.float32)
    orc.oracle().orc_nvfp4_quantize_rows(orc.p(x), x.shape[1], rows, k, static_gs, orc.p(codes), orc.p(scales), ss, orc.p(gs))
    return codes, scales, gs


@pytest.mark.parametrize("k", [512, 17408])
def test_representable_rows_come_back_bit_for_bit(k):
    """tests/cuda/moe_w4a4_test.cu:291-326: values on the grid of block scale 0.25 (amax 1.5 / 6) under a static global of 1
    decode to the same BF16 values: the scale rule and the e2m1 rounding are the checkpoint's."""
    x = nd.representable_rows(k)
    codes, scales, gs = oracle_quantize(x, x.shape[0], k, 1.0)
    assert np.all(gs == 1.0) and np.all(scales[:, :k // 16] == 0x28)            # e4m3 0.25
    back = nd.dequantize(codes, scales, gs, k)
    assert np.array_equal(nd.f32_to_bf16_bits(back.astype(np.float32)), x)


@pytest.mark.parametrize("k,static_gs", [(64, 0.0), (1024, 0.0), (1024, 0.25), (6144, 0.0), (2048, 0.003)])
def test_quantizer_matches_the_numpy_restatement(k, static_gs):
    rows = 9
    x = nd.activation_rows(rows, k, 100 + k, stride=k + 8)
    x[3, :k] = 0                                   # a zero row: global 1, everything zero
    x[4, 16:48] = 0                                # zero blocks inside a live row
    codes, scales, gs = oracle_quantize(x, rows, k, static_gs)
    want_codes, want_scales, want_gs = nd.quantize_numpy(x, k, static_gs)
    assert np.array_equal(gs.view(np.uint32), want_gs.view(np.uint32))
    assert np.array_equal(scales, want_scales), "scale bytes (padding bytes must stay untouched)"
    assert np.array_equal(codes, want_codes)
    if static_gs == 0.0:
        assert gs[3] == 1.0 and not codes[3].any() and not scales[3, :k // 16].any()
        # the decoded rows are the activations up to NVFP4 rounding: half a code step of the block's scale
        back = nd.dequantize(codes, scales, gs, k)
        xf = bf16_bits_to_f64(x[:, :k])
        step = np.repeat(nd.e4m3_decode(scales[:, :k // 16]), 16, axis=1) * gs[:, None].astype(np.float64)
        assert np.all(np.abs(back - xf) <= 1.0 * step + 1e-30)


def test_quantizer_saturates_under_a_small_static_global():
    k = 64
    x = nd.f32_to_bf16_bits(np.full((1, k), 1000.0, np.float32))
    x[0, 1] = nd.f32_to_bf16_bits(np.float32(-1000.0))
    codes, scales, gs = oracle_quantize(x, 1, k, 1e-3)          # 6 * 448 * 1e-3 = 2.7 << 1000
    assert gs[0] == np.float32(1e-3) and np.all(scales[0, :4] == 0x7E)          # the block scale saturates at 448
    assert codes[0, 0] == 0xF7 and np.all(codes[0, 1:] == 0x77)                 # codes saturate at +-6


def test_w4a4_gemm_oracle_matches_numpy():
    m, n, k = 5, 7, 128
    x = nd.activation_rows(m, k, 7)
    codes, scales, gs = oracle_quantize(x, m, k)
    rng = np.random.default_rng(3)
    wc = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    ws = nd.e4m3_encode(rng.uniform(0.05, 1.5, (n, k // 16)).astype(np.float32))
    wg = 417.0
    out, mag = np.empty((m, n)), np.empty((m, n))
    orc.oracle().orc_w4a4_gemm(orc.p(codes), orc.p(scales), scales.shape[1], orc.p(gs), orc.p(wc), orc.p(ws), wg, m, n, k,
                               orc.p(out), orc.p(mag))
    a = nd.dequantize(codes, scales, gs, k)
    w = nd.dequantize(wc, ws, np.ones(n), k) / wg
    assert np.allclose(out, a @ w.T, rtol=1e-13, atol=1e-300)
    assert np.allclose(mag, np.abs(a) @ np.abs(w).T, rtol=1e-13)


def test_launchers_refuse_bad_geometry_without_a_gpu():
    from dgpp_amd import launch as L
    fake = 0x10000
    assert L.nvfp4_act_scale_stride(512) == 32 and L.nvfp4_act_scale_stride(320) == 24 and L.nvfp4_act_scale_stride(64) == 8
    for k in (0, 32, 100, 32768 + 64):
        with pytest.raises(L.InvalidArgument):
            L.launch_quantize_rows_nvfp4(fake, 40000, 2, k, fake, fake, fake)
    with pytest.raises(L.InvalidArgument):
        L.launch_quantize_rows_nvfp4(fake + 2, 512, 2, 512, fake, fake, fake)          # misaligned rows
    with pytest.raises(L.InvalidArgument):
        L.launch_quantize_rows_nvfp4(fake, 516, 2, 512, fake, fake, fake)              # stride not a multiple of 8
    with pytest.raises(L.InvalidArgument):
        L.launch_swiglu_quantize_rows_nvfp4(fake, None, 512, 2, 512, 10.0, fake, fake, fake)
    L.launch_quantize_rows_nvfp4(None, 512, 0, 512, None, None, None)                  # rows <= 0 returns silently
    with pytest.raises(L.InvalidArgument):
        L.launch_moe_grouped_w4a4_f32(fake, fake, fake, None, fake, 3, 4, fake, 0, fake, 64, 64, 96)    # k % 64
    with pytest.raises(L.InvalidArgument):
        L.launch_moe_grouped_w4a4_f32(fake, fake, fake, None, fake, 3, 0, fake, 0, fake, 64, 64, 128)   # max_rows
    L.launch_moe_grouped_w4a4_f32(fake, fake, fake, None, fake, 0, 4, fake, 0, fake, 64, 64, 128)       # no segments


def oracle_minimax_quantize(x, rows, k):
    codes = np.empty((rows, k // 2), np.uint8)
    scales = np.empty((rows, k // 16), np.uint8)
    glob = np.empty(rows, np.float32)
    orc.oracle().orc_minimax_quantize_rows_nvfp4(orc.p(x), x.shape[1], rows, k, orc.p(codes), orc.p(scales), orc.p(glob))
    return codes, scales, glob


@pytest.mark.parametrize("k", [128, 3072, 6144])
def test_minimax_producer_matches_the_numpy_restatement(k):
    """What this pins: the restated chain (multiplications by correctly rounded reciprocals). What it cannot: the last
    bit of the reference's approximate reciprocal instruction (parity unpinned in that respect)."""
    rows = 7
    x = nd.activation_rows(rows, k, 300 + k, stride=k + 3)
    x[2, :k] = 0
    x[5, 32:64] = 0
    x[5, 40] = 0x8000                                  # a negative zero in a zero block: its sign survives in the code
    codes, scales, glob = oracle_minimax_quantize(x, rows, k)
    want = nd.minimax_quantize_numpy(x, k)
    assert np.array_equal(glob.view(np.uint32), want[2].view(np.uint32))
    assert np.array_equal(scales, want[1]) and np.array_equal(codes, want[0])
    assert glob[2] == 0.0 and not scales[2].any() and not codes[2].any()
    assert codes[5, 20] == 0x08 and not scales[5, 2:4].any()
    # the decode identity: rows come back within half a code step (one where the scale byte rounded down)
    back = nd.dequantize(codes, scales, glob, k)
    xf = bf16_bits_to_f64(x[:, :k])
    step = np.repeat(nd.e4m3_decode(scales), 16, axis=1) * glob[:, None].astype(np.float64)
    assert np.all(np.abs(back - xf) <= step + 1e-30)
    # the row maximum lands on the top code of the top scale: amax / 2688 * 448 * 6
    live = [r for r in range(rows) if r != 2]
    assert np.allclose(np.abs(back[live]).max(axis=1), np.abs(xf[live]).max(axis=1), rtol=2e-6)
    # rows do not depend on the rows beside them
    one = oracle_minimax_quantize(np.ascontiguousarray(x[4:5]), 1, k)
    assert np.array_equal(one[0][0], codes[4]) and np.array_equal(one[1][0], scales[4]) and one[2][0] == glob[4]


def test_minimax_swiglu_f32_oracle_closed_form_points():
    alpha, limit = 1.702, 7.0
    gate = np.array([0.0, 3.0, 100.0, -100.0, 2.0, 2.0, 1.0], np.float32)
    up = np.array([5.0, -1.0, 0.5, 0.5, 100.0, -100.0, 0.25], np.float32)
    out, exact = np.empty(7, np.uint16), np.empty(7)
    orc.oracle().orc_minimax_swiglu_f32(orc.p(gate), orc.p(up), 7, alpha, limit, orc.p(out), orc.p(exact))
    sig = lambda v: 1.0 / (1.0 + np.exp(-alpha * v))
    want = np.array([0.0, 0.0, 7.0 * sig(7.0) * 1.5, -100.0 * sig(-100.0) * 1.5, 2.0 * sig(2.0) * 8.0, 2.0 * sig(2.0) * -6.0,
                     sig(1.0) * 1.25])
    assert np.allclose(exact, want, rtol=1e-14, atol=1e-300)
    assert np.array_equal(out, nd.f32_to_bf16_bits(want.astype(np.float32)))


def test_minimax_and_dense_launchers_refuse_bad_geometry_without_a_gpu():
    from dgpp_amd import launch as L
    fake = 0x10000
    for k in (0, 64, 192, 32768 + 128):
        with pytest.raises(L.InvalidArgument):
            L.minimax_quantize_rows_nvfp4(fake, 40000, 2, k, fake, fake, fake)
    with pytest.raises(L.InvalidArgument):
        L.minimax_quantize_rows_nvfp4(fake, 100, 2, 128, fake, fake, fake)             # stride below k
    L.minimax_quantize_rows_nvfp4(None, 128, 0, 128, None, None, None)
    L.minimax_swiglu_f32(None, None, None, 0, 1.702, 7.0)
    with pytest.raises(L.InvalidArgument):
        L.minimax_swiglu_f32(fake, None, fake, 5, 1.702, 7.0)
    assert L.dense_w4a4_supported(128) and L.dense_w4a4_supported(6144) and not L.dense_w4a4_supported(192)
    with pytest.raises(L.InvalidArgument):
        L.launch_dense_w4a4_bf16(fake, fake, 8, fake, fake, fake, fake, fake, 64, 4, 64, 192)       # k % 128
    with pytest.raises(L.InvalidArgument):
        L.launch_dense_w4a4_bf16(fake, fake, 4, fake, fake, fake, fake, fake, 64, 4, 64, 128)       # scale stride below k / 16
    with pytest.raises(L.InvalidArgument):
        L.launch_dense_w4a4_bf16(fake, fake, 8, fake, fake, fake, fake, fake, 32, 4, 64, 128)       # out_stride below n
    with pytest.raises(L.InvalidArgument):
        L.launch_moe_accum_ordered_bf16down(fake, fake, 64, fake, fake, fake, 3, 17, 64)            # top_k above 16
