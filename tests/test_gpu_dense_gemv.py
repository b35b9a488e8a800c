"""Dense projection GEMV (NVFP4 / MXFP4 / FP8 block-scaled / MXFP8) against the CPU oracle.

Budget: the reference's strict comparator — 2 bf16 ulps with a 1e-3 * max|oracle| cancellation
floor, zero mismatches, l2_rel <= 1e-3 (tests/cuda/scale_gemm_test_helpers.hpp:72-100,
tests/cuda/fp4_gemv_test.cu:166-174) — and the north-star measure error beyond the bf16
output's own half-ulp rounding, relative to max(|oracle_fp64|, floor), <= 2e-3.
"""
import numpy as np
import pytest

import oracle_lib as orc
from dgpp_amd import hostgen as hg, launch as L
from gpu_util import dev, dev_empty, fp4_matrix, host, sync

pytestmark = pytest.mark.gpu


def make_fp4(m, n, k, seed, group, std=0.02):
    w = hg.normal_f32(seed, (n, k), std)
    act = hg.normal_bf16(seed + 1, (m, k), 1.0)
    if group == 16:
        payload, scales, ws2 = hg.encode_nvfp4(w)
        glob = np.array([1.0 / np.float32(ws2)], dtype=np.float32)
    else:
        payload, scales = hg.encode_mxfp4(w)
        glob = None
    return act, payload, scales, glob


def run_fp4(act, payload, scales, glob, group, m, n, k, f32=False):
    act_d, p_d, s_d = dev(act), dev(payload), dev(scales)
    g_d = dev(glob) if glob is not None else None
    w = fp4_matrix(p_d, s_d, g_d, n, k, group)
    out = dev_empty((m, n), np.float32 if f32 else np.uint16)
    (L.launch_fp4_gemv_f32 if f32 else L.launch_fp4_gemv_bf16)(act_d, k, w, out, m, n, k, None)
    sync()
    return host(out, np.float32 if f32 else np.uint16)


def check(got_bits, raw, label):
    # strict comparator: both sides speak bf16 (the oracle's fp64 dot rounded once)
    strict = hg.bf16_to_f32(orc.bf16_round(raw)).astype(np.float64)
    rep = orc.compare_bf16(got_bits, strict, 2.0, 1e-3)
    assert rep.nan_pattern_errors == 0, label
    assert rep.mismatches == 0, f"{label}: {rep.mismatches} mismatches, max {rep.max_ulps:.2f} ulps"
    assert rep.l2_rel <= 1e-3, f"{label}: l2_rel {rep.l2_rel}"
    # north-star measure against the UNROUNDED fp64 value (beyond bf16's own half-ulp), floor 1e-3 * max
    ns = orc.north_star_rel(got_bits, raw, 1e-3)
    assert ns <= 2e-3, f"{label}: north-star rel {ns}"


SHAPES = [(1, 520, 4096), (3, 264, 1024), (2, 100, 512), (4, 40, 256), (1, 33, 128), (2, 17, 64), (1, 9, 32),
          (4, 512, 4096), (2, 300, 2048), (1, 390, 5120), (3, 130, 5120), (2, 520, 384), (1, 77, 768), (4, 70, 1536),
          (2, 41, 3072), (1, 20, 12288), (8, 136, 6144), (5, 64, 2560),
          (16, 200, 2048), (64, 96, 4096), (37, 70, 640)]          # more rows than one vector pass: the launcher's matrix-core form


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_nvfp4_gemv_matches_oracle(gpu, m, n, k):
    act, payload, scales, glob = make_fp4(m, n, k, 0xF40 + n + k, 16)
    raw = orc.gemv_fp4(act, payload, scales, float(glob[0]), 16, m, n, k)
    check(run_fp4(act, payload, scales, glob, 16, m, n, k), raw, f"nvfp4 M{m} N{n} K{k}")


MX_SHAPES = [(1, 520, 4096), (3, 264, 1024), (2, 100, 512), (4, 40, 256), (1, 33, 128), (2, 17, 64), (1, 9, 32),
             (2, 300, 2048), (1, 390, 5120), (2, 75, 576), (1, 130, 1152), (3, 66, 2304), (8, 96, 4096),
             (16, 200, 2048), (64, 96, 4096)]


@pytest.mark.parametrize("m,n,k", MX_SHAPES)
def test_mxfp4_gemv_matches_oracle(gpu, m, n, k):
    act, payload, scales, _ = make_fp4(m, n, k, 0x3F40 + n + k, 32)
    raw = orc.gemv_fp4(act, payload, scales, 1.0, 32, m, n, k)
    check(run_fp4(act, payload, scales, None, 32, m, n, k), raw, f"mxfp4 M{m} N{n} K{k}")


def test_mxfp4_random_codes_and_wide_scale_range(gpu):
    """Random codes with random e8m0 bytes over the whole useful range (tests/cuda/fp4_gemv_test.cu:67-85
    style data), including bytes at the ends that take the exact fp32 path."""
    rng = np.random.default_rng(7)
    m, n, k = 2, 96, 1024
    payload = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    scales = rng.integers(100, 140, (n, k // 32), dtype=np.uint8)
    scales[3, 5], scales[7, 0] = 1, 0          # 2^-126 and 2^-127: the exact fp32 path
    act = hg.normal_bf16(99, (m, k))
    raw = orc.gemv_fp4(act, payload, scales, 1.0, 32, m, n, k)
    got = run_fp4(act, payload, scales, None, 32, m, n, k)
    check(got, raw, "mxfp4 random codes")
    # a row made only of tiny scales: products far below the rest, still finite and right
    scales[20, :] = rng.integers(0, 3, k // 32, dtype=np.uint8)
    raw = orc.gemv_fp4(act, payload, scales, 1.0, 32, m, n, k)
    got = run_fp4(act, payload, scales, None, 32, m, n, k)
    g20 = hg.bf16_to_f32(got[:, 20]).astype(np.float64)
    assert np.all(np.abs(g20 - raw[:, 20]) <= np.abs(raw[:, 20]) * 2.0 ** -7 + 2.0 ** -133)


@pytest.mark.parametrize("group", [16, 32])
def test_fp4_rows_are_independent_of_row_count(gpu, group):
    """tests/cuda/fp4_gemv_test.cu:342-371: a row's bits do not depend on m, for both epilogues."""
    for k in ([4096, 512, 5120, 384] if group == 16 else [4096, 512, 5120, 576]):
        act, payload, scales, glob = make_fp4(8, 136, k, 0xE8 + k, group)
        got8 = run_fp4(act, payload, scales, glob, group, 8, 136, k)
        got8f = run_fp4(act, payload, scales, glob, group, 8, 136, k, f32=True)
        assert np.array_equal(hg.f32_to_bf16(got8f), got8), "bf16(out_f32) == out_bf16"
        for r in range(8):
            one = run_fp4(act[r:r + 1], payload, scales, glob, group, 1, 136, k)
            assert np.array_equal(one[0], got8[r]), f"k={k} row {r} bits depend on m"
        got3 = run_fp4(act[:3], payload, scales, glob, group, 3, 136, k)
        assert np.array_equal(got3, got8[:3])


def test_nvfp4_nan_scales_poison_exactly_their_rows(gpu):
    act, payload, scales, glob = make_fp4(1, 300, 1024, 0xA5, 16)
    scales[9, 3] = 0x7F
    scales[250, 0] = 0xFF
    got = hg.bf16_to_f32(run_fp4(act, payload, scales, glob, 16, 1, 300, 1024))[0]
    nan = np.isnan(got)
    assert nan[9] and nan[250] and nan.sum() == 2


def test_mxfp4_nan_scales_poison_exactly_their_rows(gpu):
    act, payload, scales, _ = make_fp4(1, 300, 1024, 0x3A5, 32)
    scales[9, 3] = 0xFF
    scales[250, 0] = 0xFF
    got = hg.bf16_to_f32(run_fp4(act, payload, scales, None, 32, 1, 300, 1024))[0]
    nan = np.isnan(got)
    assert nan[9] and nan[250] and nan.sum() == 2


def test_fp4_geometry_contract(gpu):
    """tests/cuda/fp4_gemv_test.cu:276-313, 398-415."""
    def rejects(k, group):
        act, payload, scales, glob = make_fp4(1, 8, k, 0xBAD, group) if k % 32 == 0 else (
            hg.normal_bf16(1, (1, k)), np.zeros((8, k // 2), np.uint8), np.zeros((8, max(1, k // group)), np.uint8),
            np.ones(1, np.float32) if group == 16 else None)
        try:
            run_fp4(act, payload, scales, glob, group, 1, 8, k)
        except L.InvalidArgument:
            return True
        return False
    assert rejects(48, 16) and rejects(96, 16) and rejects(8192, 16)
    assert not rejects(1536, 16) and not rejects(2048, 16) and not rejects(5120, 16)
    assert rejects(48, 32) and rejects(3072, 32)
    for k in (576, 1152, 2304, 4096, 2048):
        assert not rejects(k, 32)
    # an NVFP4 view without its global is refused
    act, payload, scales, glob = make_fp4(1, 8, 1024, 0xBAE, 16)
    w = fp4_matrix(dev(payload), dev(scales), None, 8, 1024, 16)
    with pytest.raises(L.InvalidArgument):
        L.launch_fp4_gemv_bf16(dev(act), 1024, w, dev_empty((1, 8), np.uint16), 1, 8, 1024, None)


# ---- FP8 block-scaled -----------------------------------------------------------------------------------
def make_fp8(m, n, k, seed, br=128, bc=128):
    w = hg.f32_to_bf16(hg.normal_f32(seed, (n, k), 0.02))
    payload, scales = hg.encode_fp8_blocks(w, br, bc)
    act = hg.normal_bf16(seed + 1, (m, k))
    return act, payload, scales


FP8_SHAPES = [(1, 4096, 4096), (1, 520, 4096), (3, 264, 1024), (2, 100, 512), (4, 200, 768), (8, 130, 2048),
              (1, 33, 144), (2, 17, 16), (5, 260, 6144), (1, 70, 7168),
              (16, 130, 2048), (64, 96, 1024), (9, 40, 304)]           # more rows than one vector pass: the launcher's matrix-core form


@pytest.mark.parametrize("m,n,k", FP8_SHAPES)
def test_fp8_scale_gemm_matches_oracle(gpu, m, n, k):
    act, payload, scales = make_fp8(m, n, k, 0x8F0 + n + k)
    raw = orc.gemv_fp8(act, payload, scales, m, n, k, 7, 7, strict=True)
    out = dev_empty((m, n), np.uint16)
    L.launch_scale_gemm_bf16(dev(act), k, dev(payload), dev(scales), out, m, n, k, None)
    outf = dev_empty((m, n), np.float32)
    L.launch_scale_gemm_f32(dev(act), k, dev(payload), dev(scales), outf, m, n, k, None)
    sync()
    got = host(out, np.uint16)
    check(got, raw, f"fp8 M{m} N{n} K{k}")
    assert np.array_equal(hg.f32_to_bf16(host(outf)), got)
    # semantic oracle (true dequant in fp64): 8 ulps / 2e-2 floor / <= 5 % mismatches
    sem = orc.gemv_fp8(act, payload, scales, m, n, k, 7, 7, strict=False)
    rep = orc.compare_bf16(got, sem, 8.0, 2e-2)
    assert rep.mismatches <= 0.05 * rep.total


@pytest.mark.parametrize("rs,cs,br,bc", [(5, 5, 32, 32), (6, 7, 64, 128), (0, 5, 1, 32), (0, 12, 1, 4096)])
def test_fp8_scale_gemm_grid(gpu, rs, cs, br, bc):
    m, n, k = 3, 200, 1024
    act, payload, scales = make_fp8(m, n, k, 0x6A1D + rs * 8 + cs, br, min(bc, k))
    if bc > k:  # channel grid: one scale per row
        payload, scales = hg.encode_fp8_blocks(hg.f32_to_bf16(hg.normal_f32(5, (n, k), 0.02)), 1, k)
    raw = orc.gemv_fp8(act, payload, scales, m, n, k, rs, cs, strict=True)
    out = dev_empty((m, n), np.uint16)
    L.launch_scale_gemm_grid_bf16(dev(act), k, dev(payload), dev(scales), out, m, n, k, None, 0, rs, cs)
    sync()
    check(host(out, np.uint16), raw, f"fp8 grid rs{rs} cs{cs}")


def test_mxfp8_e8m0_grid(gpu):
    for (m, n, k) in [(1, 300, 6144), (8, 129, 4096), (3, 50, 96)]:
        w = hg.normal_f32(0xE8 + k, (n, k), 0.02)
        payload, scales = hg.encode_mxfp8(w)
        act = hg.normal_bf16(0xE9 + k, (m, k))
        raw = orc.gemv_fp8(act, payload, scales, m, n, k, 0, 5, strict=True, e8m0=True)
        out = dev_empty((m, n), np.uint16)
        L.launch_scale_gemm_grid_e8m0_bf16(dev(act), k, dev(payload), dev(scales), out, m, n, k, None, 0, 0, 5)
        sync()
        check(host(out, np.uint16), raw, f"mxfp8 M{m} N{n} K{k}")


def test_fp8_rows_independent_and_strided_output(gpu):
    m, n, k = 8, 136, 2048
    act, payload, scales = make_fp8(m, n, k, 0x51)
    p_d, s_d = dev(payload), dev(scales)
    out = dev_empty((m, n + 24), np.uint16)
    out.zero_()
    L.launch_scale_gemm_bf16(dev(act), k, p_d, s_d, out, m, n, k, None, n + 24)
    sync()
    full = host(out, np.uint16)
    assert not full[:, n:].any(), "columns past n stay untouched"
    for r in range(m):
        one = dev_empty((1, n), np.uint16)
        L.launch_scale_gemm_bf16(dev(act[r:r + 1]), k, p_d, s_d, one, 1, n, k, None)
        sync()
        assert np.array_equal(host(one, np.uint16)[0], full[r, :n])
    # last_row_only / compact_row write one row of the same product
    outf = dev_empty((m, n), np.float32)
    outf.zero_()
    L.launch_scale_gemm_f32(dev(act), k, p_d, s_d, outf, m, n, k, None, 0, 0, True)
    sync()
    got = host(outf)
    assert not got[:m - 1].any() and np.array_equal(hg.f32_to_bf16(got[m - 1]), full[m - 1, :n])
    L.launch_scale_gemm_f32(dev(act), k, p_d, s_d, outf, m, n, k, None, 0, 0, False, None, 0, 2)
    sync()
    assert np.array_equal(hg.f32_to_bf16(host(outf)[0]), full[2, :n])


def test_fp8_zero_k_and_argument_errors(gpu):
    out = dev_empty((2, 8), np.uint16)
    out.fill_(7)
    dummy = dev(np.zeros(16, np.uint8))
    L.launch_scale_gemm_bf16(dummy, 0, dummy, dev(np.ones(1, np.float32)), out, 2, 8, 0, None)
    sync()
    assert not host(out).any(), "k == 0 gives zeros"
    with pytest.raises(L.InvalidArgument):
        L.launch_scale_gemm_bf16(None, 16, dummy, dummy, out, 1, 8, 16, None)
    with pytest.raises(L.InvalidArgument):
        L.launch_scale_gemm_bf16(dummy, 16, dummy, dummy, out, 1, 8, 16, None, 4)  # stride below n
    with pytest.raises(L.InvalidArgument):
        L.launch_scale_gemm_grid_bf16(dummy, 16, dummy, dummy, out, 1, 8, 16, None, 0, 3, 3)


def test_fp8_dequant_bridge_is_bit_exact(gpu):
    """Every e4m3 code times a spread of scales: bf16(decode * scale) bit for bit (also proves the
    device codec is OCP E4M3FN)."""
    rows, cols = 256, 256
    payload = np.tile(np.arange(256, dtype=np.uint8), (rows, 1))
    rng = np.random.default_rng(3)
    scales = np.exp2(rng.uniform(-20, 6, (2, 2))).astype(np.float32)
    want = np.empty((rows, cols), np.float64)
    orc.oracle().orc_dequant_fp8(orc.p(payload), orc.p(scales), None, rows, cols, 7, 7, 1, orc.p(want))
    out = dev_empty((rows, cols), np.uint16)
    L.launch_fp8_dequant_blocks(dev(payload), dev(scales), out, rows, cols, None)
    sync()
    got = hg.bf16_to_f32(host(out, np.uint16)).astype(np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want[ok])


def test_fp8_gemv_multi_is_bitwise_the_single_launches(gpu):
    """launch_scale_gemv_multi_bf16 (reference: src/kernels/scale_gemm.hpp:88-107, its test
    scale_gemm_gemv_multi_is_bitwise_the_single_launches): up to four [n_i, k] matrices against the same rows, every
    out_i bitwise the single launcher's for its problem, for every row count the form takes (1 .. 8)."""
    from dgpp_amd import _lib
    k = 1024
    geo = [(264, 7, 7, 0), (100, 5, 5, 128), (520, 6, 7, 0), (48, 0, 5, 64)]     # n, rs, cs, out_stride (0: n)
    mats = []
    for i, (n, rs, cs, _) in enumerate(geo):
        w = hg.f32_to_bf16(hg.normal_f32(0x3A00 + i, (n, k), 0.02))
        payload, scales = hg.encode_fp8_blocks(w, 1 << rs, 1 << cs)
        mats.append((dev(payload), dev(scales)))
    assert L.fp8_gemv_can_stage(mats[0][0], k) and not L.fp8_gemv_can_stage(mats[0][0], k + 8)
    for rows in (1, 3, 4, 5, 8):
        act = dev(hg.normal_bf16(0x3B00 + rows, (rows, k + 16)))                 # rows strided by k + 16 elements
        outs, singles, problems = [], [], []
        for (n, rs, cs, stride), (p_d, s_d) in zip(geo, mats):
            o = dev_empty((rows, stride or n), np.uint16)
            o.zero_()
            outs.append(o)
            problems.append(_lib.Fp8GemvProblem(p_d.data_ptr(), s_d.data_ptr(), o.data_ptr(), n, 0, stride, rs, cs, None))
            one = dev_empty((rows, n), np.uint16)
            L.launch_scale_gemm_grid_bf16(act, k + 16, p_d, s_d, one, rows, n, k, None, 0, rs, cs)
            singles.append(one)
        L.launch_scale_gemv_multi_bf16(problems, act, k + 16, rows, k)
        sync()
        for (n, _, _, stride), o, one in zip(geo, outs, singles):
            got = host(o, np.uint16)
            assert np.array_equal(got[:, :n], host(one, np.uint16)), f"rows {rows}, n {n}"
            assert not got[:, n:].any(), "columns past n stay untouched"
    with pytest.raises(L.InvalidArgument):
        L.launch_scale_gemv_multi_bf16(problems + problems[:1], act, k + 16, 8, k)        # five problems
    with pytest.raises(L.InvalidArgument):
        L.launch_scale_gemv_multi_bf16(problems, act, k + 16, 9, k)                       # nine rows
    bad = _lib.Fp8GemvProblem(mats[0][0].data_ptr(), mats[0][1].data_ptr(), outs[0].data_ptr(), 264, 0, 0, 7, 7,
                              mats[0][0].data_ptr())
    with pytest.raises(L.InvalidArgument):
        L.launch_scale_gemv_multi_bf16([bad], act, k + 16, 1, k)                          # a bf16-weight problem


def test_fp8_saturation_extremes(gpu):
    """The reference's scale_gemm_saturation_extremes (tests/cuda/scale_gemm_test.cu:501-532): all-maximum payloads
    (0x7E = 448) with scales of 1e30 (products near 1e35 stay finite in bf16 and fp32), and the minimum subnormal
    (0x01 = 2^-9) with scales of 2^-20: both ends of the exponent range against both oracles."""
    m, n, k = 8, 256, 256
    for code, scale, seed, label in ((0x7E, 1e30, 0xD4, "448 x 1e30"), (0x01, 2.0 ** -20, 0xD5, "subnormal minimum")):
        payload = np.full((n, k), code, np.uint8)
        scales = np.full((2, 2), scale, np.float32)
        act = hg.normal_bf16(seed, (m, k))
        out = dev_empty((m, n), np.uint16)
        L.launch_scale_gemm_bf16(dev(act), k, dev(payload), dev(scales), out, m, n, k, None)
        sync()
        got = host(out, np.uint16)
        assert np.isfinite(hg.bf16_to_f32(got)).all(), label
        check(got, orc.gemv_fp8(act, payload, scales, m, n, k, 7, 7, strict=True), label)
        sem = orc.gemv_fp8(act, payload, scales, m, n, k, 7, 7, strict=False)
        assert orc.compare_bf16(got, sem, 8.0, 2e-2).mismatches == 0, label


def test_fp8_gemv_decodes_every_code_as_the_bridge_does(gpu):
    """The reference's fp8_gemv_hardware_conversion_matches_bridge_on_every_code: a one-hot activation reads single
    weights back through the GEMV; for every e4m3 code and a spread of block scales the value is the dequant
    bridge's bf16(decode * scale), bit for bit (NaN codes give NaN)."""
    n, k = 256, 256
    payload = np.tile(np.arange(256, dtype=np.uint8)[:, None], (1, k))          # row r holds code r everywhere
    rng = np.random.default_rng(5)
    scales = np.exp2(rng.uniform(-18, 8, (2, 2))).astype(np.float32)
    bridge = dev_empty((n, k), np.uint16)
    L.launch_fp8_dequant_blocks(dev(payload), dev(scales), bridge, n, k, None)
    cols = [3, 200]                                                             # one column in each scale block
    act = np.zeros((len(cols), k), np.uint16)
    for i, c in enumerate(cols):
        act[i, c] = 0x3F80                                                      # 1.0
    out = dev_empty((len(cols), n), np.float32)
    L.launch_scale_gemm_f32(dev(act), k, dev(payload), dev(scales), out, len(cols), n, k, None)
    sync()
    got, want = host(out), hg.bf16_to_f32(host(bridge, np.uint16))
    for i, c in enumerate(cols):
        # a NaN weight times the zeros of the other columns poisons its whole row either way: rows 0x7F and 0xFF are NaN
        nan = np.isnan(want[:, c])
        assert np.array_equal(np.isnan(got[i]), nan) and nan.sum() == 2
        # values, not bit patterns: code 0x80 (-0) leaves the dot's accumulator at +0 (0 + -0 * 1), as fmaf does
        assert np.array_equal(got[i][~nan], want[:, c][~nan]), f"column {c}"
        assert np.count_nonzero(got[i][~nan]) == 252                              # every code but the two zeros


def test_e8m0_grid_is_bitwise_the_f32_grid_of_the_same_powers_of_two(gpu):
    """The reference's mma_gemv_fp8_e8m0_grid_is_bitwise_the_f32_grid, for the GEMV launchers and the matrix-core
    launchers: an E8M0 byte grid and the F32 grid holding 2^(b - 127) describe the same weights, and every product
    e4m3 * 2^e is exact in bf16, so the two launchers give the same bits."""
    m, n, k = 5, 200, 1024
    w = hg.normal_f32(0xE80, (n, k), 0.02)
    payload, bytes_ = hg.encode_mxfp8(w)
    bytes_ = np.ascontiguousarray(bytes_)
    f32 = np.exp2(bytes_.astype(np.float64) - 127.0).astype(np.float32)
    act = dev(hg.normal_bf16(0xE81, (m, k)))
    p_d, b_d, f_d = dev(payload), dev(bytes_), dev(f32)
    a, b = dev_empty((m, n), np.uint16), dev_empty((m, n), np.uint16)
    L.launch_scale_gemm_grid_e8m0_bf16(act, k, p_d, b_d, a, m, n, k, None, 0, 0, 5)
    L.launch_scale_gemm_grid_bf16(act, k, p_d, f_d, b, m, n, k, None, 0, 0, 5)
    sync()
    assert np.array_equal(host(a, np.uint16), host(b, np.uint16)), "GEMV launchers"
    a2, b2 = dev_empty((m, n), np.float32), dev_empty((m, n), np.float32)
    L.launch_mma_gemv_fp8e8m0_f32(act, k, p_d, b_d, a2, m, n, k, 0, 0, 5, None)
    L.launch_mma_gemv_fp8_f32(act, k, p_d, f_d, b2, m, n, k, 0, 0, 5, None)
    sync()
    assert np.array_equal(host(a2).view(np.uint32), host(b2).view(np.uint32)), "matrix-core launchers"


def test_fp8_dequant_bridge_e8m0_is_bit_exact(gpu):
    """The bridge over an E8M0 byte grid (reference: src/kernels/fp8_dequant.cu:28-31, :79-83): every e4m3 code under
    block bytes across the range that keeps the products inside bf16's normal range, plus bytes 0 and 255:
    bf16(decode * 2^(b - 127)) bit for bit, NaN where the code or the byte says so."""
    rows, cols = 64, 256
    payload = np.tile(np.arange(256, dtype=np.uint8), (rows, 1))
    rng = np.random.default_rng(9)
    scales = rng.integers(20, 240, (rows, cols // 32), dtype=np.uint8)
    scales[0, 0], scales[1, 1], scales[2, 2] = 0, 255, 254
    want = np.empty((rows, cols), np.float64)
    orc.oracle().orc_dequant_fp8(orc.p(payload), None, orc.p(scales), rows, cols, 0, 5, 1, orc.p(want))
    out = dev_empty((rows, cols), np.uint16)
    L.launch_fp8_dequant_blocks_e8m0(dev(payload), dev(scales), out, rows, cols, None, 0, 5)
    sync()
    got = hg.bf16_to_f32(host(out, np.uint16)).astype(np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want[ok])
    with pytest.raises(L.InvalidArgument):
        L.launch_fp8_dequant_blocks_e8m0(dev(payload), dev(scales), out, rows, cols, None, 0, 3)
