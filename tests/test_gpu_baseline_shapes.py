"""The five benchmark configurations at their FULL shapes on the GPU: oracle checks where the CPU
finishes in seconds (whole outputs for C1 / C3 / C4, row and token samples for C2 / C5) plus
size-independent properties (rows independent of the batch, slot path == grouped path, bf16(f32) ==
bf16 epilogue). Only experts that the seeded routing selects are materialised; the remaining table
entries alias one of them (they are never read)."""
import numpy as np
import pytest

import moe_data
import oracle_lib as orc
from dgpp_amd import hostgen as hg, launch as L, moe_layer as ML
from gpu_util import dev, dev_empty, fp4_matrix, fp4_view, fp8_view, host, sync
from test_gpu_dense_gemv import check
from test_gpu_moe_slots import expert_budget

pytestmark = pytest.mark.gpu


def test_c1_dense_fp8_4096x4096(gpu):
    n = k = 4096
    w = hg.f32_to_bf16(hg.normal_f32(0xD6990010, (n, k), 0.02))
    payload, scales = hg.encode_fp8_blocks(w, 128, 128)
    act = hg.normal_bf16(0xD6990011, (1, k))
    raw = orc.gemv_fp8(act, payload, scales, 1, n, k, 7, 7, True)
    out = dev_empty((1, n), np.uint16)
    L.launch_scale_gemm_bf16(dev(act), k, dev(payload), dev(scales), out, 1, n, k, None)
    sync()
    check(host(out, np.uint16), raw, "C1")


def test_c2_dense_nvfp4_17408x5120(gpu):
    """C2 at full size. Batch 1: every one of the 17,408 rows against the fp64 oracle. Batch 8 rides the matrix-core
    form inside launch_fp4_gemv_* (row-count dispatch): its rows are bitwise the matrix-core launcher's, row blocks are
    held to the oracle, and the vector-core rows (batch 1, batch 4) agree with each other bit for bit."""
    n, k = 17408, 5120
    w = hg.normal_f32(0xD6990020, (n, k), 0.02)
    payload, scales, ws2 = hg.encode_nvfp4(w)
    del w
    glob = np.array([1.0 / np.float32(ws2)], np.float32)
    act = hg.normal_bf16(0xD6990021, (8, k))
    p_d, s_d, g_d, a_d = dev(payload), dev(scales), dev(glob), dev(act)
    wm = fp4_matrix(p_d, s_d, g_d, n, k, 16)
    out8, out8f, out1 = dev_empty((8, n), np.uint16), dev_empty((8, n), np.float32), dev_empty((1, n), np.uint16)
    out4 = dev_empty((4, n), np.uint16)
    L.launch_fp4_gemv_bf16(a_d, k, wm, out8, 8, n, k, None)
    L.launch_fp4_gemv_f32(a_d, k, wm, out8f, 8, n, k, None)
    L.launch_fp4_gemv_bf16(a_d, k, wm, out1, 1, n, k, None)
    L.launch_fp4_gemv_bf16(a_d, k, wm, out4, 4, n, k, None)
    sync()
    got8, got1 = host(out8, np.uint16), host(out1, np.uint16)
    assert np.array_equal(got1[0], host(out4, np.uint16)[0]), "batch-1 row == batch-4 row 0 (vector core), every output"
    assert np.array_equal(hg.f32_to_bf16(host(out8f)), got8)
    raw1 = orc.gemv_fp4(act[:1], payload, scales, float(glob[0]), 16, 1, n, k)      # all 17,408 rows
    check(got1, raw1, "C2 batch 1, every row")
    out8m = dev_empty((8, n), np.uint16)
    L.launch_dense_mma_fp4_bf16(a_d, k, wm, out8m, 8, n, k, None)
    sync()
    assert np.array_equal(host(out8m, np.uint16), got8), "batch 8: launch_fp4_gemv == the matrix-core launcher, bit for bit"
    for r0 in (0, 8192, n - 1024):          # row blocks against the oracle (rows are independent)
        sl = slice(r0, r0 + 1024)
        raw = orc.gemv_fp4(act, np.ascontiguousarray(payload[sl]), np.ascontiguousarray(scales[sl]), float(glob[0]),
                           16, 8, 1024, k)
        check(np.ascontiguousarray(got8[:, sl]), raw, f"C2 batch 8 rows {r0}")


def _used_experts_table(ids, E, make_views):
    """views list of E*3 entries: selected experts get their own weights, the rest alias the first."""
    used = sorted(set(int(v) for v in ids.ravel()))
    per = {e: make_views(e) for e in used}
    views = []
    for e in range(E):
        views += per.get(e, per[used[0]])[0]
    return views, per


def test_c3_mxfp4_moe_decode_layer(gpu):
    E, H, I, K, T = 256, 4096, 1024, 8, 8
    x = hg.normal_bf16(0xD6990030, (T, H))
    logits = hg.bf16_to_f32(hg.normal_bf16(0xD6990031, (T, E)))
    l64 = logits.astype(np.float64)
    ids, w = np.empty((T, K), np.int32), np.empty((T, K), np.float32)
    orc.oracle().orc_router_select(orc.p(l64), orc.p(l64), 1, T, E, K, 1.0, 1, orc.p(ids), orc.p(w))
    keep = []

    def make(e):
        mats = [moe_data.make_mat("mxfp4", I, H, 0xD6993000 + e * 3), moe_data.make_mat("mxfp4", I, H, 0xD6993001 + e * 3),
                moe_data.make_mat("mxfp4", H, I, 0xD6993002 + e * 3)]
        vs = []
        for m in mats:
            pd, sd = dev(m.payload), dev(m.scales)
            keep.extend([pd, sd])
            vs.append(fp4_view(pd, sd, None, 32))
        return vs, mats

    views, per = _used_experts_table(ids, E, make)
    cfg = L.make_config(H, I, E, K, n_shared_experts=0, routed_scaling_factor=1.0, swiglu_limit=float("inf"),
                        router_mode=L.ROUTER_SOFTMAX_TOPK)
    layer = ML.MoeLayer(cfg, ML.EXPERTS_MXFP4, views, T)
    x_d, lg_d = dev(x), dev(logits)
    experts = [per[e][1] if e in per else per[int(ids[0, 0])][1] for e in range(E)]
    orc_experts = [m.orc() for e in experts for m in e]
    prev = None
    for t in (1, 4, 8):
        out = dev_empty((t, H), np.uint16)
        layer.enqueue_decode_scores(x_d, H, lg_d, lg_d, out, t)
        outg = dev_empty((t, H), np.uint16)
        layer.enqueue_grouped_routed(x_d, H, dev(ids[:t]), dev(w[:t]), outg, t)
        sync()
        got = host(out, np.uint16)
        assert np.array_equal(got, host(outg, np.uint16)), "decode slots == grouped path, bitwise"
        raw, _ = orc.moe_forward(x[:t], ids[:t], w[:t], H, I, I, orc_experts, None, float("inf"), threads=8)
        expert_budget(got, raw, f"C3 T={t}")
        if prev is not None:
            assert np.array_equal(got[:prev.shape[0]], prev), "a token's output does not depend on the batch"
        prev = got
    layer.close()


def test_c4_fp8_moe_zipf(gpu):
    E, H, I, K, T = 128, 2048, 768, 8, 32
    ids = hg.zipf_routes(0xD6990040, 1.1, T, K, E)
    lg = hg.normal_f32(0xD6990041, (T, K)).astype(np.float64)
    pw = np.exp(lg - lg.max(axis=1, keepdims=True))
    w = (pw / pw.sum(axis=1, keepdims=True)).astype(np.float32)      # renormalised softmax of N(0,1)
    x = hg.normal_bf16(0xD6990042, (T, H))
    keep = []

    def make(e):
        mats = [moe_data.make_mat("fp8", I, H, 0xD6994000 + e * 3), moe_data.make_mat("fp8", I, H, 0xD6994001 + e * 3),
                moe_data.make_mat("fp8", H, I, 0xD6994002 + e * 3)]
        vs = []
        for m in mats:
            pd, sd = dev(m.payload), dev(m.scales)
            keep.extend([pd, sd])
            vs.append(fp8_view(pd, sd, 7, 7))
        return vs, mats

    views, per = _used_experts_table(ids, E, make)
    counts = np.bincount(ids.ravel(), minlength=E)
    assert counts.max() >= 8, "the Zipf routing must produce busy experts (skewed tokens per expert)"
    cfg = L.make_config(H, I, E, K, n_shared_experts=0, routed_scaling_factor=1.0, swiglu_limit=float("inf"),
                        router_mode=L.ROUTER_SOFTMAX_TOPK)
    layer = ML.MoeLayer(cfg, ML.EXPERTS_FP8, views, T)
    x_d, ids_d, w_d = dev(x), dev(ids), dev(w)
    out, outg = dev_empty((T, H), np.uint16), dev_empty((T, H), np.uint16)
    layer.enqueue_decode_routed(x_d, H, ids_d, w_d, out, T)
    layer.enqueue_grouped_routed(x_d, H, ids_d, w_d, outg, T)
    sync()
    got = host(out, np.uint16)
    assert np.array_equal(got, host(outg, np.uint16))
    first = per[int(ids[0, 0])][1]
    orc_experts = [m.orc() for e in range(E) for m in (per[e][1] if e in per else first)]
    raw, _ = orc.moe_forward(x, ids, w, H, I, I, orc_experts, None, float("inf"), threads=8)
    expert_budget(got, raw, "C4")
    outm = dev_empty((T, H), np.uint16)
    layer.enqueue_prefill_routed(x_d, H, ids_d, w_d, outm, T)
    sync()
    expert_budget(host(outm, np.uint16), raw, "C4, matrix-core grouped path")
    # grouping tables of the same routing, bit-exact against the host counting sort
    rows, slot_row, segs = np.empty(T * K + T, np.int32), np.empty(T * K, np.int32), np.empty((E + 1, 3), np.int32)
    orc.oracle().orc_moe_segment(orc.p(ids), T, K, E, orc.p(rows), orc.p(slot_row), orc.p(segs))
    rows_d, sr_d, segs_d = dev_empty(T * K + T, np.int32), dev_empty(T * K, np.int32), dev_empty((E + 1, 3), np.int32)
    L.launch_moe_segment(ids_d, T, K, E, rows_d, sr_d, segs_d, None)
    sync()
    assert np.array_equal(host(rows_d), rows) and np.array_equal(host(sr_d), slot_row) and np.array_equal(host(segs_d), segs)
    layer.close()


def test_c5_nvfp4_routed_plus_mxfp8_shared(gpu):
    """C5 at full size. The whole layer is ONE call of the layer driver (NVFP4 routed experts in decode slots, the MXFP8
    shared expert of its own width as dense projections beside them, combined last with weight 1): bitwise the chain
    stitched from the loose launchers, and held to the oracle on twelve tokens spread over the batch whose routes reach
    at least 32 distinct generated experts. The same layer is then routed by the MiniMax router from an FP32 gate
    (routes and FP32 weights equal the oracle's bit for bit) and six of its tokens are held to the oracle."""
    E, H, I, K, T, SI = 256, 6144, 2048, 8, 64, 4096
    BASE, G = 10, 40                         # BASE generated experts; expert e uses variant e % G of them (variant g is
                                             # base expert g % BASE with its rows rotated by 64 * (g // BASE): other weights)
    x = hg.normal_bf16(0xD6990050, (T, H))
    logits = hg.bf16_to_f32(hg.normal_bf16(0xD6990051, (T, E)))
    l64 = logits.astype(np.float64)
    ids, w = np.empty((T, K), np.int32), np.empty((T, K), np.float32)
    orc.oracle().orc_router_select(orc.p(l64), orc.p(l64), 1, T, E, K, 1.0, 1, orc.p(ids), orc.p(w))
    keep, gen, base = [], [], []
    for b in range(BASE):
        base.append([moe_data.make_mat("nvfp4", I, H, 0xD6995000 + b * 3), moe_data.make_mat("nvfp4", I, H, 0xD6995001 + b * 3),
                     moe_data.make_mat("nvfp4", H, I, 0xD6995002 + b * 3)])
    for g in range(G):
        shift = 64 * (g // BASE)
        mats = [moe_data.Mat(m.kind, m.rows, m.cols, np.ascontiguousarray(np.roll(m.payload, shift, axis=0)),
                             np.ascontiguousarray(np.roll(m.scales, shift, axis=0)), m.glob) if shift else m
                for m in base[g % BASE]]
        vs = []
        for m in mats:
            pd, sd, gd = dev(m.payload), dev(m.scales), dev(m.glob)
            keep.extend([pd, sd, gd])
            vs.append(fp4_view(pd, sd, gd, 16))
        gen.append((vs, mats))
    views = [v for e in range(E) for v in gen[e % G][0]]
    cfg = L.make_config(H, I, E, K, n_shared_experts=0, routed_scaling_factor=1.0, swiglu_limit=float("inf"),
                        router_mode=L.ROUTER_SOFTMAX_TOPK)
    layer = ML.MoeLayer(cfg, ML.EXPERTS_NVFP4, views, T)
    x_d, lg_d = dev(x), dev(logits)
    routed = dev_empty((T, H), np.float32)
    layer.enqueue_decode_scores(x_d, H, lg_d, lg_d, None, T, out_f32=routed)
    routed_g = dev_empty((T, H), np.float32)
    layer.enqueue_grouped_routed(x_d, H, dev(ids), dev(w), None, T, out_f32=routed_g)
    sync()
    assert np.array_equal(host(routed), host(routed_g)), "decode slots == grouped path, bitwise"
    # the shared MXFP8 expert (weight 1, last in the chain): dense E8M0-grid projections at m = 64
    sh = [moe_data.make_mat("mxfp8", SI, H, 0xD6995900), moe_data.make_mat("mxfp8", SI, H, 0xD6995901),
          moe_data.make_mat("mxfp8", H, SI, 0xD6995902)]
    shd = [(dev(m.payload), dev(m.scales)) for m in sh]
    g_d, u_d, a_d = (dev_empty((T, SI), np.uint16) for _ in range(3))
    L.launch_scale_gemm_grid_e8m0_bf16(x_d, H, shd[0][0], shd[0][1], g_d, T, SI, H, None, 0, 0, 5)
    L.launch_scale_gemm_grid_e8m0_bf16(x_d, H, shd[1][0], shd[1][1], u_d, T, SI, H, None, 0, 0, 5)
    L.launch_moe_swiglu_clamp(g_d, u_d, a_d, T * SI, float("inf"), None)
    shared_down = dev_empty((T, H), np.float32)
    L.launch_scale_gemm_grid_e8m0_f32(a_d, SI, shd[2][0], shd[2][1], shared_down, T, H, SI, None, 0, 0, 5)
    # continue the chain: acc = fma(1, shared, routed), one rounding
    rows_id = dev(np.arange(T, dtype=np.int32))
    L.launch_moe_accum(routed, shared_down, rows_id, dev(np.ones(T, np.float32)), T, H, None)
    out = dev_empty((T, H), np.uint16)
    L.launch_moe_round_bf16(out, routed, T * H, None)
    sync()
    got = host(out, np.uint16)
    assert np.array_equal(hg.f32_to_bf16(host(routed_g) + host(shared_down)), got), "fma(1, shared, acc) == acc + shared"
    # the same layer as ONE driver call: a layer whose shared expert is the dense MXFP8 form
    cfg1 = L.make_config(H, I, E, K, n_shared_experts=1, routed_scaling_factor=1.0, swiglu_limit=float("inf"),
                         router_mode=L.ROUTER_SOFTMAX_TOPK)
    layer1 = ML.MoeLayer(cfg1, ML.EXPERTS_NVFP4, views, T, shared_inter=SI, sh_payload=[t[0] for t in shd],
                         sh_scales_e8m0=[t[1] for t in shd])
    out1 = dev_empty((T, H), np.uint16)
    layer1.enqueue_decode_scores(x_d, H, lg_d, lg_d, out1, T)
    sync()
    assert np.array_equal(host(out1, np.uint16), got), "one driver call == the chain stitched from the launchers, bitwise"
    out1b = dev_empty((13, H), np.uint16)       # a smaller batch through the same layer, given routes
    layer1.enqueue_decode_routed(x_d, H, dev(ids[:13]), dev(w[:13]), out1b, 13)
    sync()
    assert np.array_equal(host(out1b, np.uint16), got[:13]), "rows do not depend on the batch they ride in"
    # the same layer routed by its donor family's router (src/kernels/minimax.hpp:56-60: FP32 gate, sigmoid scores, the
    # bias in the ranking only, FP32 weights never narrowed): routes equal the oracle's, six tokens against the oracle
    rng = np.random.default_rng(0xC5)
    gate = (rng.normal(0, 1.0, (E, H)) / np.sqrt(H)).astype(np.float32)
    bias = rng.normal(0, 0.1, E).astype(np.float32)
    sc_d, ids_d, w_d = dev_empty((T, E), np.float32), dev_empty((T, K), np.int32), dev_empty((T, K), np.float32)
    L.minimax_router(x_d, dev(gate), dev(bias), T, H, E, K, 2.5, sc_d, ids_d, w_d)
    out_mm = dev_empty((T, H), np.uint16)
    layer1.enqueue_decode_routed(x_d, H, ids_d, w_d, out_mm, T)
    sync()
    scores_mm = np.ascontiguousarray(host(sc_d, np.float32))
    ids_mm, w_mm = np.empty((T, K), np.int32), np.empty((T, K), np.float32)
    orc.oracle().orc_minimax_route_scores(orc.p(scores_mm), orc.p(bias), T, E, K, 2.5, orc.p(ids_mm), orc.p(w_mm))
    assert np.array_equal(host(ids_d, np.int32), ids_mm), "MiniMax routes"
    assert np.array_equal(host(w_d, np.float32).view(np.uint32), w_mm.view(np.uint32)), "MiniMax weights, FP32 bit for bit"
    layer1.close()
    sample_mm = [1, 14, 27, 39, 50, 62]
    orc_experts_mm = [m.orc() for e in range(E) for m in gen[e % G][1]]
    raw_mm, _ = orc.moe_forward(np.ascontiguousarray(x[sample_mm]), np.ascontiguousarray(ids_mm[sample_mm]),
                                np.ascontiguousarray(w_mm[sample_mm]), H, I, SI, orc_experts_mm, [m.orc() for m in sh],
                                float("inf"), threads=8)
    expert_budget(np.ascontiguousarray(host(out_mm, np.uint16)[sample_mm]), raw_mm, "C5 routed by the MiniMax router")
    # twelve tokens against the oracle (routed NVFP4 chain + MXFP8 shared expert)
    sample = [0, 5, 11, 17, 23, 29, 34, 40, 46, 52, 58, 63]
    assert len({int(e) % G for e in ids[sample].ravel()}) >= 32, "the sampled tokens must reach >= 32 distinct generated experts"
    orc_experts = [m.orc() for e in range(E) for m in gen[e % G][1]]
    raw, _ = orc.moe_forward(np.ascontiguousarray(x[sample]), np.ascontiguousarray(ids[sample]),
                             np.ascontiguousarray(w[sample]), H, I, SI, orc_experts, [m.orc() for m in sh],
                             float("inf"), threads=8)
    expert_budget(np.ascontiguousarray(got[sample]), raw, "C5 sampled tokens")
    # the same layer through the matrix-core launchers: routed experts by the grouped form with the gather folded
    # in, the shared expert by the E8M0-grid form at m = 64 (four 16-row tiles per weight pass)
    routed_m = dev_empty((T, H), np.float32)
    layer.enqueue_prefill_routed(x_d, H, dev(ids), dev(w), None, T, out_f32=routed_m)
    L.launch_mma_gemv_fp8e8m0_bf16(x_d, H, shd[0][0], shd[0][1], g_d, T, SI, H, 0, 0, 5, None)
    L.launch_mma_gemv_fp8e8m0_bf16(x_d, H, shd[1][0], shd[1][1], u_d, T, SI, H, 0, 0, 5, None)
    L.launch_moe_swiglu_clamp(g_d, u_d, a_d, T * SI, float("inf"), None)
    L.launch_mma_gemv_fp8e8m0_f32(a_d, SI, shd[2][0], shd[2][1], shared_down, T, H, SI, 0, 0, 5, None)
    L.launch_moe_accum(routed_m, shared_down, rows_id, dev(np.ones(T, np.float32)), T, H, None)
    out_m = dev_empty((T, H), np.uint16)
    L.launch_moe_round_bf16(out_m, routed_m, T * H, None)
    sync()
    expert_budget(np.ascontiguousarray(host(out_m, np.uint16)[sample]), raw, "C5 sampled tokens, matrix-core launchers")
    counts = np.bincount(ids.ravel(), minlength=E)
    print(f"C5 routing: {np.count_nonzero(counts)} distinct experts, busiest {counts.max()} tokens")
    layer.close()
