"""The matrix-core launchers (dense, scale-grid and grouped forms) against the CPU oracle, and the
properties the reference pins for its tensor-core kernels (tests/cuda/glm_moe_test.cu grouped-vs-dense
per segment, tests/cuda/scale_gemm_test.cu:255-330 rows bitwise the rows alone): a (weight row,
activation row) result does not depend on how many rows ride in the launch, on the launcher, or on the
split form. Budget: the strict single-GEMV comparator of test_gpu_dense_gemv.check.
"""
import numpy as np
import pytest

import moe_data
import oracle_lib as orc
from dgpp_amd import _lib, hostgen as hg, launch as L
from gpu_util import DeviceMoe, dev, dev_empty, fp4_matrix, host, sync
from test_gpu_dense_gemv import check, make_fp4

pytestmark = pytest.mark.gpu

FP4_SHAPES = [(1, 520, 4096), (5, 200, 1024), (16, 100, 2048), (37, 130, 5120), (8, 64, 160), (3, 33, 576),
              (20, 77, 6144), (2, 16, 32)]


@pytest.mark.parametrize("group", [16, 32])
@pytest.mark.parametrize("m,n,k", FP4_SHAPES)
def test_dense_mma_fp4_matches_oracle_and_rows_are_independent(gpu, group, m, n, k):
    act, payload, scales, glob = make_fp4(m, n, k, 0x3A0 + n + k + group, group)
    raw = orc.gemv_fp4(act, payload, scales, float(glob[0]) if glob is not None else 1.0, group, m, n, k)
    act_d, p_d, s_d = dev(act), dev(payload), dev(scales)
    g_d = dev(glob) if glob is not None else None
    w = fp4_matrix(p_d, s_d, g_d, n, k, group)
    out, outf, one = dev_empty((m, n), np.uint16), dev_empty((m, n), np.float32), dev_empty((1, n), np.uint16)
    L.launch_dense_mma_fp4_bf16(act_d, k, w, out, m, n, k, None)
    L.launch_dense_mma_fp4_f32(act_d, k, w, outf, m, n, k, None)
    last = act_d[m - 1:m].contiguous()
    L.launch_dense_mma_fp4_bf16(last, k, w, one, 1, n, k, None)
    outs = dev_empty((m, n + 8), np.uint16)
    ws = dev_empty(4 * m * n, np.float32)
    L.launch_mma_gemv_fp4_bf16(act_d, k, w, outs, m, n, k, n + 8, None, ws, 4 * m * n * 4)
    outsf = dev_empty((m, n + 8), np.float32)
    L.launch_mma_gemv_fp4_f32(act_d, k, w, outsf, m, n, k, n + 8, None, ws, 4 * m * n * 4)
    sync()
    got = host(out, np.uint16)
    assert np.array_equal(host(outs, np.uint16)[:, :n], got), "the split form's bits are the unsplit form's"
    assert np.array_equal(hg.f32_to_bf16(host(outsf)[:, :n]), got), "the split form's unrounded output rounds to the same bits"
    check(got, raw, f"dense mma fp4 g{group} {m}x{n}x{k}")
    assert np.array_equal(hg.f32_to_bf16(host(outf)), got), "bf16(out_f32) == out_bf16"
    assert np.array_equal(host(one, np.uint16)[0], got[m - 1]), "a row's bits do not depend on the rows beside it"


@pytest.mark.parametrize("e8m0,rs,cs", [(False, 7, 7), (False, 5, 6), (False, 0, 12), (True, 0, 5)])
@pytest.mark.parametrize("m,n,k", [(1, 300, 4096), (9, 130, 2048), (33, 96, 1024), (16, 50, 304), (64, 128, 6144)])
def test_mma_gemv_fp8_matches_oracle_split_and_unsplit(gpu, e8m0, rs, cs, m, n, k):
    if e8m0 and k % 32:
        k -= k % 32                      # the 1 x 32 grid needs whole blocks
    rng = np.random.default_rng(n + k + rs)
    w = hg.f32_to_bf16(hg.normal_f32(0x8A0 + n + k, (n, k), 0.02))
    act = hg.normal_bf16(0x8A1 + n, (m, k))
    if e8m0:
        payload, scales = hg.encode_mxfp8(hg.bf16_to_f32(w))
    else:
        payload, _ = hg.encode_fp8_blocks(w, 128, 128)
        br, bc = 1 << rs, 1 << cs
        scales = rng.uniform(0.5, 2.0, ((n + br - 1) // br, (k + bc - 1) // bc)).astype(np.float32) * 1e-3
    raw = orc.gemv_fp8(act, payload, scales, m, n, k, rs, cs, True, e8m0)
    a_d, p_d, s_d = dev(act), dev(payload), dev(scales)
    fn_b = L.launch_mma_gemv_fp8e8m0_bf16 if e8m0 else L.launch_mma_gemv_fp8_bf16
    fn_f = L.launch_mma_gemv_fp8e8m0_f32 if e8m0 else L.launch_mma_gemv_fp8_f32
    stride = n + 8
    out, outf, outs = dev_empty((m, stride), np.uint16), dev_empty((m, n), np.float32), dev_empty((m, n), np.uint16)
    out.zero_()
    ws = dev_empty(4 * m * n, np.float32)
    fn_b(a_d, k, p_d, s_d, out, m, n, k, stride, rs, cs, None)
    fn_f(a_d, k, p_d, s_d, outf, m, n, k, 0, rs, cs, None)
    fn_b(a_d, k, p_d, s_d, outs, m, n, k, 0, rs, cs, None, ws, 4 * m * n * 4)
    sync()
    got = host(out, np.uint16)
    assert not got[:, n:].any(), "columns past n are left alone"
    got = np.ascontiguousarray(got[:, :n])
    check(got, raw, f"mma gemv fp8 e8m0={e8m0} {m}x{n}x{k} rs{rs} cs{cs}")
    assert np.array_equal(hg.f32_to_bf16(host(outf)), got)
    assert np.array_equal(host(outs, np.uint16), got), "the split form's bits are the unsplit form's"
    if not e8m0 and rs == 7 and cs == 7:
        outd, outdf = dev_empty((m, n), np.uint16), dev_empty((m, n), np.float32)
        L.launch_dense_mma_bf16(a_d, k, p_d, s_d, outd, m, n, k, None)
        L.launch_dense_mma_f32(a_d, k, p_d, s_d, outdf, m, n, k, None)
        sync()
        assert np.array_equal(host(outd, np.uint16), got)
        assert np.array_equal(hg.f32_to_bf16(host(outdf)), got)


@pytest.mark.parametrize("kind", ["fp8", "nvfp4", "mxfp4"])
def test_grouped_mma_is_bitwise_the_dense_mma_per_segment_with_and_without_the_gather(gpu, kind):
    E, H, I, K, T = 6, 512, 160 if kind != "fp8" else 144, 3, 23          # segments of up to 23 rows: two tiles
    p = moe_data.make_problem(E, H, I, K, T, kind, 41, shared_kind=None, limit=float("inf"), std=0.05)
    d = DeviceMoe(p)
    ids, w, _, _ = moe_data.orc_router(p, 1, 1.0, True)
    ids_d = dev(ids)
    rows_d, sr_d, segs_d = dev_empty(T * K + T, np.int32), dev_empty(T * K, np.int32), dev_empty((E + 1, 3), np.int32)
    L.launch_moe_segment(ids_d, T, K, E, rows_d, sr_d, segs_d, None)
    xg = dev_empty((T * K, H), np.uint16)
    L.launch_moe_gather_rows(d.x, rows_d, xg, T * K, H, None)
    g1, g2, g3 = (dev_empty((T * K, I), np.uint16) for _ in range(3))
    gf = dev_empty((T * K, I), np.float32)
    if kind == "fp8":
        L.launch_moe_grouped_mma_bf16(xg, H, segs_d, E, T, 0, d.views, 0, g1, I, I, H, None)
        L.launch_moe_grouped_mma_bf16(d.x, H, segs_d, E, T, 0, d.views, 0, g2, I, I, H, None, rows_d)
        L.launch_moe_grouped_mma_bf16(xg, H, segs_d, E, T, 16, d.views, 0, g3, I, I, H, None)
        L.launch_moe_grouped_mma_f32(xg, H, segs_d, E, T, 0, d.views, 0, gf, I, I, H, None)
    else:
        L.launch_moe_grouped_mma_fp4_bf16(xg, H, segs_d, E, T, 0, d.views, 0, g1, I, I, H, None, None, d.fp4_group)
        L.launch_moe_grouped_mma_fp4_bf16(d.x, H, segs_d, E, T, 0, d.views, 0, g2, I, I, H, None, rows_d, d.fp4_group)
        L.launch_moe_grouped_mma_fp4_bf16(xg, H, segs_d, E, T, 16, d.views, 0, g3, I, I, H, None, None, d.fp4_group)
        L.launch_moe_grouped_mma_fp4_f32(xg, H, segs_d, E, T, 0, d.views, 0, gf, I, I, H, None, None, d.fp4_group)
    sync()
    a = host(g1, np.uint16)
    assert np.array_equal(a, host(g2, np.uint16)), "the folded gather reads the gathered buffer's values"
    assert np.array_equal(a, host(g3, np.uint16)), "the z split does not change a row"
    assert np.array_equal(hg.f32_to_bf16(host(gf)), a)
    segs, rows = host(segs_d).reshape(-1, 3), host(rows_d)
    xh = host(xg, np.uint16)
    for e in range(E):
        r0, cnt, _ = (int(v) for v in segs[e])
        if cnt == 0:
            continue
        m = p.experts[e][0]
        xs = dev(xh[r0:r0 + cnt])
        one = dev_empty((cnt, I), np.uint16)
        if kind == "fp8":
            L.launch_dense_mma_bf16(xs, H, dev(m.payload), dev(m.scales), one, cnt, I, H, None)
            raw = orc.gemv_fp8(xh[r0:r0 + cnt], m.payload, m.scales, cnt, I, H, 7, 7, True)
        else:
            wm = fp4_matrix(dev(m.payload), dev(m.scales), dev(m.glob) if m.glob is not None else None, I, H, d.fp4_group)
            L.launch_dense_mma_fp4_bf16(xs, H, wm, one, cnt, I, H, None)
            raw = orc.gemv_fp4(xh[r0:r0 + cnt], m.payload, m.scales, float(m.glob[0]) if m.glob is not None else 1.0,
                               d.fp4_group, cnt, I, H)
        sync()
        assert np.array_equal(host(one, np.uint16), a[r0:r0 + cnt]), f"segment {e}: grouped == dense, bitwise"
        check(np.ascontiguousarray(a[r0:r0 + cnt]), raw, f"grouped mma {kind} segment {e}")


@pytest.mark.parametrize("m,n,k,limit", [(3, 200, 1024, 7.0), (20, 96, 2048, float("inf")), (16, 130, 304, 0.5)])
def test_mma_gemv_fp8_swiglu_is_bitwise_swiglu_then_mma_gemv(gpu, m, n, k, limit):
    """src/kernels/mma_gemv.hpp:86-95: the activation computed as the rows are staged gives the bits of
    launch_moe_swiglu_clamp followed by launch_mma_gemv_fp8_f32 (unsplit)."""
    w = hg.f32_to_bf16(hg.normal_f32(0x9A0 + n + k, (n, k), 0.02))
    payload, scales = hg.encode_fp8_blocks(w, 128, 128)
    gate, up = hg.normal_bf16(0x9A1 + n, (m, k), 2.0), hg.normal_bf16(0x9A2 + n, (m, k))
    g_d, u_d, p_d, s_d = dev(gate), dev(up), dev(payload), dev(scales)
    act, want, got = dev_empty((m, k), np.uint16), dev_empty((m, n), np.float32), dev_empty((m, n), np.float32)
    L.launch_moe_swiglu_clamp(g_d, u_d, act, m * k, limit, None)
    _lib.load().dgpp_tune_set(5, 2)      # the comparison runs on the matrix core at every row count, as the fused form does
    try:
        L.launch_mma_gemv_fp8_f32(act, k, p_d, s_d, want, m, n, k, 0, 7, 7, None)
    finally:
        _lib.load().dgpp_tune_set(5, 0)
    L.launch_mma_gemv_fp8_swiglu_f32(g_d, u_d, limit, k, p_d, s_d, got, m, n, k, 0, 7, 7, None)
    sync()
    assert np.array_equal(host(got).view(np.uint32), host(want).view(np.uint32))
    with pytest.raises(L.InvalidArgument):
        L.launch_mma_gemv_fp8_swiglu_f32(g_d, None, limit, k, p_d, s_d, got, m, n, k, 0, 7, 7, None)


@pytest.mark.parametrize("kind", ["nvfp4", "mxfp4"])
def test_dense_mma_fp4_prod_and_gate_up_are_the_grouped_kernel_on_one_segment(gpu, kind):
    """src/kernels/glm_moe.cu:4809-4823 and src/kernels/dense_fp4_decode.cu:310-319: one device-resident segment
    through the grouped matrix-core kernel; the paired launcher gives the bits of two prod launches."""
    E, H, I, K, T = 4, 512, 96, 2, 19
    p = moe_data.make_problem(E, H, I, K, T, kind, 55, shared_kind=None, limit=float("inf"), std=0.05)
    d = DeviceMoe(p)
    expert, m = 2, 19
    seg = dev(np.array([[0, m, expert]], np.int32))
    g1, u1, g2, u2, gg = (dev_empty((m, I), np.uint16) for _ in range(5))
    L.launch_dense_mma_fp4_prod_bf16(d.x, H, seg, d.views, 0, g1, m, I, H, None, d.fp4_group)
    L.launch_dense_mma_fp4_prod_bf16(d.x, H, seg, d.views, 1, u1, m, I, H, None, d.fp4_group)
    L.launch_dense_mma_fp4_gate_up_bf16(d.x, H, seg, d.views, g2, u2, m, I, H, None, d.fp4_group)
    L.launch_moe_grouped_mma_fp4_bf16(d.x, H, seg, 1, m, 0, d.views, 0, gg, I, I, H, None, None, d.fp4_group)
    from dgpp_amd import _lib
    for form in (1, 2):   # both forms of the paired kernel (wavefronts walking both matrices / split into gate and up walkers)
        g3, u3 = dev_empty((m, I), np.uint16), dev_empty((m, I), np.uint16)
        _lib.load().dgpp_tune_set(14, form)
        try:
            L.launch_dense_mma_fp4_gate_up_bf16(d.x, H, seg, d.views, g3, u3, m, I, H, None, d.fp4_group)
        finally:
            _lib.load().dgpp_tune_set(14, 0)
        sync()
        assert np.array_equal(host(g3, np.uint16), host(g2, np.uint16)) and np.array_equal(host(u3, np.uint16), host(u2, np.uint16))
    sync()
    assert np.array_equal(host(g1, np.uint16), host(gg, np.uint16))
    assert np.array_equal(host(g1, np.uint16), host(g2, np.uint16)) and np.array_equal(host(u1, np.uint16), host(u2, np.uint16))
    mat = p.experts[expert][1]
    raw = orc.gemv_fp4(p.x, mat.payload, mat.scales, float(mat.glob[0]) if mat.glob is not None else 1.0, d.fp4_group, m, I, H)
    check(host(u2, np.uint16), raw, f"dense mma fp4 gate_up {kind}: up rows")


@pytest.mark.parametrize("kind,limit", [("fp8", 7.0), ("nvfp4", float("inf")), ("mxfp4", 0.75)])
def test_grouped_mma_gate_up_swiglu_is_bitwise_the_three_launches(gpu, kind, limit):
    """The one-launch extension (gate rows, up rows, SwiGLU in the matrix-core grouped kernel) against the two grouped
    launches and launch_moe_swiglu_clamp, with the folded gather and with a z split."""
    E, H, I, K, T = 5, 640, 160 if kind != "fp8" else 144, 2, 21
    p = moe_data.make_problem(E, H, I, K, T, kind, 77, shared_kind=None, limit=limit, std=0.05)
    d = DeviceMoe(p)
    ids, w, _, _ = moe_data.orc_router(p, 1, 1.0, True)
    ids_d = dev(ids)
    rows_d, sr_d, segs_d = dev_empty(T * K + T, np.int32), dev_empty(T * K, np.int32), dev_empty((E + 1, 3), np.int32)
    L.launch_moe_segment(ids_d, T, K, E, rows_d, sr_d, segs_d, None)
    gate, up, want, got, got_z = (dev_empty((T * K, I), np.uint16) for _ in range(5))
    if kind == "fp8":
        L.launch_moe_grouped_mma_bf16(d.x, H, segs_d, E, T, 0, d.views, 0, gate, I, I, H, None, rows_d)
        L.launch_moe_grouped_mma_bf16(d.x, H, segs_d, E, T, 0, d.views, 1, up, I, I, H, None, rows_d)
        L.launch_moe_grouped_mma_gate_up_swiglu(d.x, H, segs_d, E, T, 0, d.views, got, I, I, H, limit, None, rows_d)
        L.launch_moe_grouped_mma_gate_up_swiglu(d.x, H, segs_d, E, T, 16, d.views, got_z, I, I, H, limit, None, rows_d)
    else:
        L.launch_moe_grouped_mma_fp4_bf16(d.x, H, segs_d, E, T, 0, d.views, 0, gate, I, I, H, None, rows_d, d.fp4_group)
        L.launch_moe_grouped_mma_fp4_bf16(d.x, H, segs_d, E, T, 0, d.views, 1, up, I, I, H, None, rows_d, d.fp4_group)
        L.launch_moe_grouped_mma_gate_up_swiglu_fp4(d.x, H, segs_d, E, T, 0, d.views, got, I, I, H, limit, None, rows_d,
                                                    d.fp4_group)
        L.launch_moe_grouped_mma_gate_up_swiglu_fp4(d.x, H, segs_d, E, T, 16, d.views, got_z, I, I, H, limit, None, rows_d,
                                                    d.fp4_group)
    L.launch_moe_swiglu_clamp(gate, up, want, T * K * I, limit, None)
    sync()
    assert np.array_equal(host(got, np.uint16), host(want, np.uint16))
    assert np.array_equal(host(got_z, np.uint16), host(want, np.uint16)), "the z split does not change a row"
    # both forms of the fused kernel: every wavefront walking gate and up in turn (1), and the block's wavefronts split
    # into gate walkers and up walkers (2; what a small grid takes by itself)
    from dgpp_amd import _lib
    for form in (1, 2):
        again = dev_empty((T * K, I), np.uint16)
        _lib.load().dgpp_tune_set(14, form)
        try:
            if kind == "fp8":
                L.launch_moe_grouped_mma_gate_up_swiglu(d.x, H, segs_d, E, T, 0, d.views, again, I, I, H, limit, None, rows_d)
            else:
                L.launch_moe_grouped_mma_gate_up_swiglu_fp4(d.x, H, segs_d, E, T, 0, d.views, again, I, I, H, limit, None, rows_d,
                                                            d.fp4_group)
        finally:
            _lib.load().dgpp_tune_set(14, 0)
        sync()
        assert np.array_equal(host(again, np.uint16), host(want, np.uint16)), f"fused gate + up form {form}"
    with pytest.raises(L.InvalidArgument):
        L.launch_moe_grouped_mma_gate_up_swiglu(d.x, H, segs_d, E, 0, 0, d.views, got, I, I, H, limit, None, rows_d)


@pytest.mark.parametrize("kind", ["fp8", "nvfp4", "mxfp4"])
def test_prefill_path_matches_oracle_and_gemv_launchers_on_the_matrix_core_are_its_twins(gpu, kind):
    """The layer's matrix-core grouped path against the oracle's layer budget; then, with the bench switch that
    moves the GEMV launchers onto the matrix core, the decode-slot kernels give the same bits as that path."""
    from dgpp_amd import moe_layer as ML
    from test_gpu_moe_layer import make_layer
    from test_gpu_moe_slots import expert_budget, run_slot_path
    E, H, I, K, T = 10, 2048, 256, 4, 21
    p = moe_data.make_problem(E, H, I, K, T, kind, 58, shared_kind=None, limit=float("inf"), std=0.05)
    d = DeviceMoe(p)
    ids, w, _, _ = moe_data.orc_router(p, 1, 1.0, True)
    layer = make_layer(p, d, 1, 1.0, T)
    out = dev_empty((T, H), np.uint16)
    layer.enqueue_prefill_routed(d.x, H, dev(ids), dev(w), out, T)
    sync()
    got = host(out, np.uint16)
    raw, _ = moe_data.orc_forward(p, ids, w)
    expert_budget(got, raw, f"prefill {kind}")
    lib = _lib.load()
    lib.dgpp_tune_set(5, 2)
    try:
        _, _, out_slots = run_slot_path(p, d, ids, w)
    finally:
        lib.dgpp_tune_set(5, 0)
    assert np.array_equal(out_slots, got), "slot kernels on the matrix core == grouped matrix-core path, bitwise"
    layer.close()


@pytest.mark.parametrize("m,n,k,rs,cs", [(33, 96, 1024, 7, 7), (5, 130, 2048, 5, 6), (64, 64, 304, 7, 7)])
def test_scale_gemm_tile_is_the_matrix_core_dense_form(gpu, m, n, k, rs, cs):
    """src/kernels/scale_gemm.hpp:173-180: the tile form of the scale GEMM; bitwise launch_mma_gemv_fp8_* (unsplit)."""
    rng = np.random.default_rng(n + k)
    w = hg.f32_to_bf16(hg.normal_f32(0x7A0 + n + k, (n, k), 0.02))
    act = hg.normal_bf16(0x7A1 + n, (m, k))
    payload, _ = hg.encode_fp8_blocks(w, 128, 128)
    br, bc = 1 << rs, 1 << cs
    scales = rng.uniform(0.5, 2.0, ((n + br - 1) // br, (k + bc - 1) // bc)).astype(np.float32) * 1e-3
    a_d, p_d, s_d = dev(act), dev(payload), dev(scales)
    tb, tf, want = dev_empty((m, n), np.uint16), dev_empty((m, n), np.float32), dev_empty((m, n), np.uint16)
    L.launch_scale_gemm_tile_bf16(a_d, k, p_d, s_d, tb, m, n, k, None, rs, cs)
    L.launch_scale_gemm_tile_f32(a_d, k, p_d, s_d, tf, m, n, k, None, rs, cs)
    _lib.load().dgpp_tune_set(5, 2)      # the matrix-core form at every row count
    try:
        L.launch_mma_gemv_fp8_bf16(a_d, k, p_d, s_d, want, m, n, k, 0, rs, cs, None)
    finally:
        _lib.load().dgpp_tune_set(5, 0)
    sync()
    got = host(tb, np.uint16)
    assert np.array_equal(got, host(want, np.uint16))
    assert np.array_equal(hg.f32_to_bf16(host(tf)), got)
    check(got, orc.gemv_fp8(act, payload, scales, m, n, k, rs, cs, True), f"scale gemm tile {m}x{n}x{k}")


def test_try_dense_fp4_decode_follows_the_shape_rule(gpu):
    """src/kernels/dense_fp4_decode.cu:297-308: inside the rule the launch is the production form's (same bits), outside
    it nothing is launched and the call says so."""
    assert L.dense_fp4_decode_shape(16, 17408, 5120) and L.dense_fp4_decode_shape(1, 64, 128)
    assert not L.dense_fp4_decode_shape(17, 64, 128) and not L.dense_fp4_decode_shape(4, 64, 192)
    assert not L.dense_fp4_decode_shape(4, 17409, 128) and not L.dense_fp4_decode_shape(4, 64, 128, 32)
    E, H, I, m = 2, 1024, 192, 11
    p = moe_data.make_problem(E, H, I, 1, m, "nvfp4", 19, shared_kind=None, limit=float("inf"), std=0.05)
    d = DeviceMoe(p)
    seg = dev(np.array([[0, m, 1]], np.int32))
    want, got = dev_empty((m, I), np.uint16), dev_empty((m, I), np.uint16)
    got.fill_(0x1234)
    L.launch_dense_mma_fp4_prod_bf16(d.x, H, seg, d.views, 1, want, m, I, H, None, 16)
    assert L.try_dense_fp4_decode_bf16(d.x, H, seg, d.views, 1, got, m, I, H, None, 16) is True
    sync()
    assert np.array_equal(host(got, np.uint16), host(want, np.uint16))
    got.fill_(0x1234)
    assert L.try_dense_fp4_decode_bf16(d.x, H, seg, d.views, 1, got, m, I, H - 64, None, 16) is False      # k % 128
    sync()
    assert np.all(host(got, np.uint16) == 0x1234), "nothing was launched"


@pytest.mark.parametrize("m,n0,n1,k,with_ws", [(1, 1536, 576, 7168, True), (8, 200, 130, 2048, False), (20, 96, 300, 1024, True),
                                                (32, 64, 64, 4096, True)])
def test_fp8_pair_launch_is_bitwise_the_two_single_launches(gpu, m, n0, n1, k, with_ws):
    """src/kernels/mma_gemv.hpp:119-130: two projections in one launch, each row's chain its single launch's."""
    acts = [hg.normal_bf16(0x6B0 + i + n0, (m, k)) for i in range(2)]
    mats = []
    for i, n in enumerate((n0, n1)):
        w = hg.f32_to_bf16(hg.normal_f32(0x6C0 + i + n + k, (n, k), 0.02))
        mats.append(hg.encode_fp8_blocks(w, 128, 128))
    a_d = [dev(a) for a in acts]
    w_d = [(dev(p), dev(s)) for p, s in mats]
    ws_floats = 4 * m * (n0 + n1)
    ws = dev_empty(ws_floats, np.float32) if with_ws else None
    outs = [dev_empty((m, n + 8), np.uint16) for n in (n0, n1)]
    want = [dev_empty((m, n + 8), np.uint16) for n in (n0, n1)]
    for t in outs + want:
        t.zero_()
    if with_ws:
        assert L.mma_gemv_pair_ok(w_d[0][0], w_d[1][0], a_d[0], a_d[1], k, m, n0, n1, k, ws, ws_floats * 4)
    assert not L.mma_gemv_pair_ok(w_d[0][0], w_d[1][0], a_d[0], a_d[1], k, m, n0, n1, k, None, 0)
    assert not L.mma_gemv_pair_ok(w_d[0][0], w_d[1][0], a_d[0], a_d[1], k, 33, n0, n1, k, ws, ws_floats * 4 if ws is not None else 0)
    assert L.mma_gemv_shape_ok(w_d[0][0], a_d[0], k, m, k) and not L.mma_gemv_shape_ok(w_d[0][0], a_d[0], k, m, k + 16)
    L.launch_mma_gemv_fp8_bf16_pair(a_d[0], w_d[0][0], w_d[0][1], outs[0], n0, n0 + 8, a_d[1], w_d[1][0], w_d[1][1], outs[1], n1,
                                    n1 + 8, k, m, k, 7, 7, None, ws, ws_floats * 4 if with_ws else 0)
    for i, n in enumerate((n0, n1)):
        L.launch_mma_gemv_fp8_bf16(a_d[i], k, w_d[i][0], w_d[i][1], want[i], m, n, k, n + 8, 7, 7, None)
    sync()
    for i, n in enumerate((n0, n1)):
        g = host(outs[i], np.uint16)
        assert np.array_equal(g, host(want[i], np.uint16)), f"problem {i}"
        check(np.ascontiguousarray(g[:, :n]), orc.gemv_fp8(acts[i], mats[i][0], mats[i][1], m, n, k, 7, 7, True), f"pair problem {i}")


@pytest.mark.parametrize("kind,shared,sI", [("fp8", "fp8", 384), ("nvfp4", "fp8", 128), ("nvfp4", "nvfp4", 256),
                                            ("mxfp4", "mxfp4", 256), ("nvfp4", "mxfp8", 192)])
def test_prefill_path_with_a_shared_expert(gpu, kind, shared, sI):
    """The layer's matrix-core grouped path with the shared expert riding along (the reference's shared_seg,
    src/models/glm/moe_layer.cpp:1293-1296, 1335-1336): a table entry joins the routed launches as segment n_experts, a
    block-FP8 expert of its own width takes its own launches, the MXFP8 form runs as dense projections beside. Held to
    the oracle's layer budget, and bitwise the decode-slot chain of the same layer with its kernels on the matrix core."""
    from dgpp_amd import moe_layer as ML
    from test_gpu_moe_layer import make_layer
    from test_gpu_moe_slots import expert_budget
    E, H, I, K, T = 10, 1024, 256, 4, 19
    p = moe_data.make_problem(E, H, I, K, T, kind, 91, shared_kind=shared, shared_I=sI, limit=7.0, std=0.05)
    ids, w, _, _ = moe_data.orc_router(p, 1, 1.0, True)
    if shared == "mxfp8":
        routed_only = moe_data.MoeProblem(E, H, I, K, T, kind, None, I, experts=p.experts, x=p.x, limit=p.limit)
        d = DeviceMoe(routed_only)
        views = list((L.MoeExpertView * (d.views.numel() // 96)).from_buffer_copy(bytes(host(d.views))))
        shd = [(dev(m.payload), dev(m.scales)) for m in p.shared]
        cfg = L.make_config(H, I, E, K, n_shared_experts=1, routed_scaling_factor=1.0, swiglu_limit=p.limit, router_mode=1)
        layer = ML.MoeLayer(cfg, ML.EXPERTS_NVFP4, views, T, shared_inter=sI, sh_payload=[t[0] for t in shd],
                            sh_scales_e8m0=[t[1] for t in shd])
    else:
        d = DeviceMoe(p)
        layer = make_layer(p, d, 1, 1.0, T)
    ids_d, w_d = dev(ids), dev(w)
    out, out2 = dev_empty((T, H), np.uint16), dev_empty((T, H), np.uint16)
    layer.enqueue_prefill_routed(d.x, H, ids_d, w_d, out, T)
    sync()
    got = host(out, np.uint16)
    raw, _ = moe_data.orc_forward(p, ids, w)
    expert_budget(got, raw, f"prefill {kind} + shared {shared}")
    lib = _lib.load()
    lib.dgpp_tune_set(5, 2)
    try:
        layer.enqueue_decode_routed(d.x, H, ids_d, w_d, out2, T)
        sync()
    finally:
        lib.dgpp_tune_set(5, 0)
    assert np.array_equal(host(out2, np.uint16), got), "decode-slot chain on the matrix core == grouped matrix-core path, bitwise"
    # the whole step from the hidden rows: the layer routes on the device, then runs the same chain over its own routes
    out3, out4 = dev_empty((T, H), np.uint16), dev_empty((T, H), np.uint16)
    if shared != "mxfp8":   # (that layer was built without a router gate)
        layer.enqueue_prefill(d.x, H, out3, T)
        layer.enqueue_prefill_routed(d.x, H, layer.ids_ptr, layer.weights_ptr, out4, T)
        sync()
        assert np.array_equal(host(out3, np.uint16), host(out4, np.uint16)) and host(out3, np.uint16).any()
        expert_budget(host(out3, np.uint16), raw, f"prefill from the hidden rows {kind} + shared {shared}")
        # the same in phases: the router over two row blocks, the chain, the accumulation per block
        out5 = dev_empty((T, H), np.uint16)
        out5.fill_(0x7F7F)
        cut = 7
        layer.route_prefill_rows(d.x, H, cut, T - cut)
        layer.route_prefill_rows(d.x, H, 0, cut)
        layer.enqueue_prefill_phased(d.x, H, T)
        layer.accumulate_prefill_rows(out5, T, cut, T - cut)
        layer.accumulate_prefill_rows(out5, T, 0, cut)
        sync()
        assert np.array_equal(host(out5, np.uint16), host(out3, np.uint16)), "phased == whole"
        with pytest.raises(L.InvalidArgument):
            layer.accumulate_prefill_rows(out5, T, T - 2, 5)
    else:
        with pytest.raises(L.InvalidArgument):
            layer.enqueue_prefill_phased(d.x, H, T)
    layer.close()


@pytest.mark.parametrize("kind,m,n,k", [("fp8", 9, 200, 4096), ("e8m0", 64, 130, 6144), ("nvfp4", 8, 530, 5120), ("mxfp4", 16, 64, 4096),
                                        ("nvfp4", 3, 48, 8192), ("mxfp4", 8, 16500, 4096), ("fp8", 16, 20470, 4096)])
def test_parts_of_k_side_by_side_in_a_block_give_the_row_tile_forms_bits(gpu, kind, m, n, k):
    """The dense matrix-core launch without a workspace that gives each of the four parts of K to its own wavefronts
    of a block and folds them in LDS (four row groups per block, or two for up to eight rows): the bits of the form
    that walks the parts one after the other, whatever the bench switch or the automatic rule picks."""
    lib = _lib.load()
    w = hg.normal_f32(0x7EA0 + n + k, (n, k), 0.02)
    act = hg.normal_bf16(0x7EA1 + n, (m, k))
    a_d = dev(act)
    if kind in ("fp8", "e8m0"):
        payload, scales = hg.encode_mxfp8(w) if kind == "e8m0" else hg.encode_fp8_blocks(hg.f32_to_bf16(w), 128, 128)
        p_d, s_d = dev(payload), dev(scales)
        fn = L.launch_mma_gemv_fp8e8m0_f32 if kind == "e8m0" else L.launch_mma_gemv_fp8_f32
        rs, cs = (0, 5) if kind == "e8m0" else (7, 7)

        def run(out):
            fn(a_d, k, p_d, s_d, out, m, n, k, 0, rs, cs, None)
    else:
        if kind == "nvfp4":
            payload, scales, ws2 = hg.encode_nvfp4(w)
            g_d = dev(np.array([1.0 / np.float32(ws2)], np.float32))
        else:
            (payload, scales), g_d = hg.encode_mxfp4(w), None
        p_d, s_d = dev(payload), dev(scales)
        wm = fp4_matrix(p_d, s_d, g_d, n, k, 16 if kind == "nvfp4" else 32)

        def run(out):
            L.launch_mma_gemv_fp4_f32(a_d, k, wm, out, m, n, k, 0, None)
    outs = {}
    lib.dgpp_tune_set(5, 2)
    try:
        for knob in (1, 0, 2, 3) if m <= 8 else (1, 0, 2):   # 0: the automatic rule
            lib.dgpp_tune_set(11, knob)
            outs[knob] = dev_empty((m, n), np.float32)
            outs[knob].fill_(-7.0)
            run(outs[knob])
        sync()
    finally:
        lib.dgpp_tune_set(11, 0)
        lib.dgpp_tune_set(5, 0)
    want = host(outs[1])
    assert np.all(want != -7.0)
    for knob, o in outs.items():
        assert np.array_equal(host(o).view(np.uint32), want.view(np.uint32)), f"switch {knob}"
