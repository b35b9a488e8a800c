"""Router, grouping and accumulation kernels against the oracle. Integer outputs are bit-exact;
the fp32 chains are bit-exact given their inputs; router weights / SwiGLU carry the reference's
own budgets (tests/cuda/qwen_moe_test.cu:105-196, tests/cuda/glm_moe_test.cu:1588)."""
import numpy as np
import pytest

import oracle_lib as orc
from dgpp_amd import hostgen as hg, launch as L
from gpu_util import dev, dev_empty, host, sync

pytestmark = pytest.mark.gpu


def routes(rng, T, K, E):
    return np.stack([np.sort(rng.choice(E, K, replace=False)) for _ in range(T)]).astype(np.int32)


@pytest.mark.parametrize("T,K,E", [(1, 8, 256), (4, 8, 256), (8, 8, 256), (32, 8, 128), (64, 8, 256), (7, 3, 5),
                                   (3, 1, 2), (300, 8, 64), (1, 16, 1024)])
def test_segment_bit_exact(gpu, T, K, E):
    rng = np.random.default_rng(T * 131 + K)
    ids = routes(rng, T, K, E)
    rows, slot_row, segs = np.empty(T * K + T, np.int32), np.empty(T * K, np.int32), np.empty((E + 1, 3), np.int32)
    orc.oracle().orc_moe_segment(orc.p(ids), T, K, E, orc.p(rows), orc.p(slot_row), orc.p(segs))
    rows_d, sr_d, segs_d = dev_empty(T * K + T, np.int32), dev_empty(T * K, np.int32), dev_empty((E + 1, 3), np.int32)
    for _ in range(2):  # second run: determinism, no state left behind
        rows_d.fill_(-1); sr_d.fill_(-1); segs_d.fill_(-1)
        L.launch_moe_segment(dev(ids), T, K, E, rows_d, sr_d, segs_d, None)
        sync()
        assert np.array_equal(host(rows_d), rows) and np.array_equal(host(sr_d), slot_row)
        assert np.array_equal(host(segs_d), segs)


def test_segment_argument_errors(gpu):
    d = dev(np.zeros(64, np.int32))
    for bad in [dict(top_k=17), dict(top_k=0), dict(n_experts=1025), dict(n_experts=0)]:
        kw = dict(top_k=8, n_experts=16)
        kw.update(bad)
        with pytest.raises(L.InvalidArgument):
            L.launch_moe_segment(d, 2, kw["top_k"], kw["n_experts"], d, d, d, None)


@pytest.mark.parametrize("T,K,E,early", [(1, 8, 256, 0), (4, 8, 256, 0), (8, 8, 256, 0), (8, 8, 64, 1), (5, 2, 3, 1),
                                         (30, 8, 16, 0), (113, 8, 8, 0), (2, 8, 256, 1)])
def test_slot_order_bit_exact(gpu, T, K, E, early):
    rng = np.random.default_rng(T * 17 + K + early)
    ids = routes(rng, T, K, E)
    slots = T * (K + 1)
    order = np.empty(slots, np.int32)
    runs = np.empty(slots + L.moe_run_groups_max(slots), np.int32)
    orc.oracle().orc_moe_slot_order(orc.p(ids), slots, K, E, early, orc.p(order), orc.p(runs))
    order_d, runs_d = dev_empty(slots, np.int32), dev_empty(runs.size, np.int32)
    L.launch_moe_slot_order(dev(ids), order_d, slots, K, E, None, bool(early), runs_d)
    sync()
    assert np.array_equal(host(order_d), order) and np.array_equal(host(runs_d), runs)
    order_d.fill_(-1)
    L.launch_moe_slot_order(dev(ids), order_d, slots, K, E, None, bool(early), None)
    sync()
    assert np.array_equal(host(order_d), order)
    with pytest.raises(L.InvalidArgument):
        L.launch_moe_slot_order(dev(ids), order_d, 1025, K, E, None)


def test_tile_list_and_compaction_bit_exact(gpu):
    rng = np.random.default_rng(9)
    for E in (37, 257, 1024):
        counts = rng.integers(0, 40, E)
        counts[rng.integers(0, E, E // 3)] = 0
        segs = np.stack([np.cumsum(counts) - counts, counts, np.arange(E)], axis=1).astype(np.int32)
        total = int(counts.sum())
        for tile_rows in (1, 16, 64):
            cap = L.moe_tile_list_capacity(E, total, tile_rows)
            want = np.zeros((cap, 2), np.int32)
            n = orc.oracle().orc_moe_tile_list(orc.p(segs), E, tile_rows, orc.p(want))
            tiles_d, count_d = dev_empty((cap, 2), np.int32), dev_empty(1, np.int32)
            L.launch_moe_tile_list(dev(segs), E, tile_rows, tiles_d, count_d, None)
            sync()
            assert int(host(count_d)[0]) == n and np.array_equal(host(tiles_d)[:n], want[:n])
        for cap in sorted({E, max(1, E // 2), 5}):
            want = np.full((cap, 3), -1, np.int32)
            orc.oracle().orc_compact_segments(orc.p(segs), orc.p(want), E, cap)
            out_d = dev_empty((cap, 3), np.int32)
            out_d.fill_(-1)
            L.minimax_compact_segments(dev(segs), out_d, E, cap, None)
            sync()
            assert np.array_equal(host(out_d), want)
    with pytest.raises(L.InvalidArgument):
        L.minimax_compact_segments(dev(segs), dev(segs), 8, 9, None)


@pytest.mark.parametrize("mode,E,K,T", [(1, 256, 8, 8), (1, 128, 8, 32), (0, 288, 8, 4), (2, 64, 6, 5), (1, 5, 2, 3),
                                        (0, 1000, 16, 2), (1, 1000, 8, 3), (0, 2048, 8, 2), (1, 4096, 16, 2)])
def test_router_select_ids_exact_weights_close(gpu, mode, E, K, T):
    """Ids are bit-exact given the scores. The weights are NOT a bit-exact contract: the device computes the softmax and
    the renormalisation in fp32 (as the reference's kernel does) while the oracle (as the reference's CPU oracle) works
    in double, so a softmax-mode weight - a bf16 value - may land on the neighbouring bf16 code when the exact value
    sits next to a rounding boundary. The test bounds every weight by one bf16 ulp, counts such flips and holds them
    to a small share; the other modes' unrounded fp32 weights stay within 2e-6 relative."""
    rng = np.random.default_rng(E + K)
    if mode == 1:   # softmax: bf16-rounded logits in both rows
        scores = hg.bf16_to_f32(hg.normal_bf16(E * 3 + T, (T, E)))
        biased = scores.copy()
    else:
        scores = rng.uniform(0.05, 0.95, (T, E)).astype(np.float32)
        biased = (scores + rng.normal(0, 0.05, (T, E))).astype(np.float32)
    scaling = 1.0 if mode == 1 else 2.5
    want_ids, want_w = np.empty((T, K), np.int32), np.empty((T, K), np.float32)
    s64, b64 = scores.astype(np.float64), biased.astype(np.float64)
    orc.oracle().orc_router_select(orc.p(s64), orc.p(b64), mode, T, E, K, scaling, 1, orc.p(want_ids), orc.p(want_w))
    cfg = L.make_config(64, 64, E, K, router_mode=mode, routed_scaling_factor=scaling, n_shared_experts=0)
    ids_d, w_d = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32)
    L.launch_moe_router_select(dev(scores), dev(biased), ids_d, w_d, cfg, T, None)
    sync()
    assert np.array_equal(host(ids_d), want_ids), "router ids must be bit-exact given the scores"
    got_w = host(w_d)
    if mode == 1:   # bf16 values within one bf16 ulp, rows sum to ~1
        assert np.array_equal(hg.bf16_to_f32(hg.f32_to_bf16(got_w)), got_w)
        assert np.all(np.abs(got_w - want_w) <= np.abs(want_w) * 2.0 ** -7)
        assert np.all(np.abs(got_w.sum(axis=1) - 1) < 0.02)
        flips = int(np.count_nonzero(got_w != want_w))
        print(f"softmax router weights E={E} K={K} T={T}: {flips} of {got_w.size} differ from the double oracle by one bf16 code")
        assert flips <= max(1, got_w.size // 16)
    else:
        assert np.allclose(got_w, want_w, rtol=2e-6, atol=0)


def test_router_tie_rule_and_full_router(gpu):
    # all-equal scores: ids 0..K-1 (tests/cuda/glm_moe_test.cu:1498-1545)
    E, K, T, H = 40, 8, 3, 256
    scores = np.full((T, E), 0.5, np.float32)
    cfg = L.make_config(H, 64, E, K, routed_scaling_factor=2.5)
    ids_d, w_d = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32)
    L.launch_moe_router_select(dev(scores), dev(scores.copy()), ids_d, w_d, cfg, T, None)
    sync()
    assert np.array_equal(host(ids_d), np.tile(np.arange(K, dtype=np.int32), (T, 1)))
    assert np.allclose(host(w_d), 0.5 / (K * 0.5) * 2.5, rtol=1e-6)
    # full router (dots + select) in the three modes, near-tie certified against the oracle's biased scores
    for mode in (0, 1, 2):
        E, K, T, H = 96, 8, 6, 512
        x = hg.normal_bf16(mode + 1, (T, H))
        gate = hg.normal_bf16(mode + 9, (E, H), 1.0 / np.sqrt(H))
        bias = hg.normal_f32(mode + 5, (E,), 0.02)
        scaling = 1.0 if mode == 1 else 2.5
        sc, bi = np.empty((T, E)), np.empty((T, E))
        orc.oracle().orc_router_scores(orc.p(x), orc.p(gate), orc.p(bias), mode, T, E, H, orc.p(sc), orc.p(bi))
        want_ids, want_w = np.empty((T, K), np.int32), np.empty((T, K), np.float32)
        orc.oracle().orc_router_select(orc.p(sc), orc.p(bi), mode, T, E, K, scaling, 1, orc.p(want_ids), orc.p(want_w))
        cfg = L.make_config(H, 64, E, K, router_mode=mode, routed_scaling_factor=scaling)
        ids_d, w_d = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32)
        sc_d, bi_d = dev_empty((T, E), np.float32), dev_empty((T, E), np.float32)
        L.launch_moe_router(dev(x), dev(gate), None if mode == 1 else dev(bias), ids_d, w_d, sc_d, bi_d, cfg, T, None)
        sync()
        got_bi = host(bi_d).astype(np.float64)
        tol = 2.0 ** -7 if mode == 1 else 1e-5        # softmax: one bf16 ulp of the logit
        assert np.all(np.abs(got_bi - bi) <= tol * np.maximum(np.abs(bi), 1e-3))
        got_ids = host(ids_d)
        for t in range(T):
            if not np.array_equal(got_ids[t], want_ids[t]):   # a swap must be a near-tie in the oracle
                a = set(got_ids[t]) ^ set(want_ids[t])
                gap = max(bi[t, list(a)]) - min(bi[t, list(a)])
                assert gap <= (2.0 ** -7 * abs(bi[t, list(a)]).max() if mode == 1 else 1e-5), (mode, t, gap)
            else:
                assert np.all(np.abs(host(w_d)[t] - want_w[t]) <= np.abs(want_w[t]) * (2.0 ** -7 if mode == 1 else 1e-4))
        with pytest.raises(L.InvalidArgument):
            L.launch_moe_router(dev(x), dev(gate), None, ids_d, w_d, sc_d, sc_d, cfg, T, None)  # aliasing
        # the dots alone, then the selection from them: the router's own bits
        sc2, bi2 = dev_empty((T, E), np.float32), dev_empty((T, E), np.float32)
        ids2, w2 = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32)
        L.launch_moe_router_dots(dev(x), dev(gate), None if mode == 1 else dev(bias), sc2, bi2, cfg, T, None)
        L.launch_moe_router_select(sc2, bi2, ids2, w2, cfg, T, None)
        sync()
        assert np.array_equal(host(sc2).view(np.uint32), host(sc_d).view(np.uint32))
        assert np.array_equal(host(bi2).view(np.uint32), host(bi_d).view(np.uint32))
        assert np.array_equal(host(ids2), got_ids) and np.array_equal(host(w2).view(np.uint32), host(w_d).view(np.uint32))
        with pytest.raises(L.InvalidArgument):
            L.launch_moe_router_dots(dev(x), dev(gate), None, sc2, sc2, cfg, T, None)           # aliasing


def test_swiglu_clamp(gpu):
    n = 70000
    g = hg.normal_bf16(1, (n,), 4.0)
    u = hg.normal_bf16(2, (n,), 6.0)
    g[:8] = hg.f32_to_bf16(np.array([0, 20, -20, 1, -1, 9, 100, 0.5], np.float32))
    u[:8] = hg.f32_to_bf16(np.array([1, 1, 1, 20, -20, -3, 2, 0.25], np.float32))
    for limit in (10.0, float("inf")):
        want = np.empty(n, np.uint16)
        orc.oracle().orc_swiglu(orc.p(g), orc.p(u), n, limit, orc.p(want))
        out = dev_empty(n, np.uint16)
        L.launch_moe_swiglu_clamp(dev(g), dev(u), out, n, limit, None)
        sync()
        got = host(out, np.uint16)
        gf, wf = hg.bf16_to_f32(got).astype(np.float64), hg.bf16_to_f32(want).astype(np.float64)
        # fp32 expf against the oracle's double: at most one bf16 ulp, almost always equal
        assert np.all(np.abs(gf - wf) <= np.abs(wf) * 2.0 ** -7 + 1e-38)
        assert np.mean(got == want) > 0.995


def test_gather_accum_round_bit_exact(gpu):
    rng = np.random.default_rng(4)
    for hidden in (4096, 100):
        src = hg.normal_bf16(3, (40, hidden))
        rows = rng.integers(0, 40, 77).astype(np.int32)
        dst = dev_empty((77, hidden), np.uint16)
        L.launch_moe_gather_rows(dev(src), dev(rows), dst, 77, hidden, None)
        sync()
        assert np.array_equal(host(dst, np.uint16), src[rows])
    T, H = 9, 300
    acc = rng.normal(size=(T, H)).astype(np.float32)
    y = rng.normal(size=(5, H)).astype(np.float32)
    rows = np.array([3, 0, 8, 1, 5], np.int32)      # distinct: one fma per output element
    w = rng.uniform(0, 1, 5).astype(np.float32)
    acc_d = dev(acc)
    L.launch_moe_accum(acc_d, dev(y), dev(rows), dev(w), 5, H, None)
    out = dev_empty((T, H), np.uint16)
    L.launch_moe_round_bf16(out, acc_d, T * H, None)
    sync()
    want = acc.copy()
    for r in range(5):
        want[rows[r]] = (w[r].astype(np.float64) * y[r].astype(np.float64) + acc[rows[r]].astype(np.float64)).astype(np.float32)
    assert np.array_equal(host(acc_d), want)
    assert np.array_equal(host(out, np.uint16), hg.f32_to_bf16(want))


@pytest.mark.parametrize("T,H,K", [(1, 4096, 8), (8, 4096, 8), (5, 333, 3), (64, 6144, 8)])
def test_slot_accum_and_ordered_accum_bit_exact(gpu, T, H, K):
    rng = np.random.default_rng(T + H)
    contrib = rng.normal(size=(T * (K + 1), H)).astype(np.float32)
    w = rng.uniform(0, 1, (T, K)).astype(np.float32)
    f32_want, bf_want = np.empty((T, H), np.float32), np.empty((T, H), np.uint16)
    orc.oracle().orc_slot_accum(orc.p(contrib), orc.p(w), T, H, K, 1, orc.p(f32_want), orc.p(bf_want))
    out = dev_empty((T, H), np.uint16)
    L.launch_moe_slot_accum(out, dev(contrib), dev(w), T, H, K, None)
    sync()
    assert np.array_equal(host(out, np.uint16), bf_want)
    orc.oracle().orc_slot_accum(orc.p(contrib), orc.p(w), T, H, K, 0, orc.p(f32_want), None)
    outf = dev_empty((T, H), np.float32)
    L.launch_moe_slot_accum_routed_f32(outf, dev(contrib), dev(w), T, H, K, None)
    sync()
    assert np.array_equal(host(outf), f32_want)
    L.launch_moe_slot_accum_routed_bf16(out, dev(contrib), dev(w), T, H, K, None)   # the fused form
    sync()
    assert np.array_equal(host(out, np.uint16), hg.f32_to_bf16(f32_want))
    # grouped layout: rows found through slot_row, slots visited in ascending expert id
    ids = np.stack([rng.permutation(64)[:K] for _ in range(T)]).astype(np.int32)
    slot_row = rng.permutation(T * K).astype(np.int32)
    down = rng.normal(size=(T * K + T, H + 8)).astype(np.float32)
    sw = rng.uniform(0, 1, T * K).astype(np.float32)
    for shared_row0 in (T * K, -1):
        orc.oracle().orc_accum_ordered(orc.p(down), H + 8, orc.p(slot_row), orc.p(ids), orc.p(sw), shared_row0, T, K, H,
                                       orc.p(f32_want), orc.p(bf_want))
        L.launch_moe_accum_ordered(out, dev(down), H + 8, dev(slot_row), dev(ids), dev(sw), shared_row0, T, K, H, None)
        L.launch_moe_accum_ordered_f32(outf, dev(down), H + 8, dev(slot_row), dev(ids), dev(sw), shared_row0, T, K, H, None)
        sync()
        assert np.array_equal(host(out, np.uint16), bf_want) and np.array_equal(host(outf), f32_want)


@pytest.mark.parametrize("mode,E,K,T,early", [(1, 256, 8, 8, False), (1, 256, 8, 1, False), (0, 288, 8, 5, True),
                                              (0, 40, 4, 16, False), (1, 512, 16, 3, False), (1, 600, 8, 4, False),
                                              (0, 64, 8, 40, False)])
def test_router_select_order_is_bitwise_select_then_slot_order(gpu, mode, E, K, T, early):
    """The one-launch extension (selection + slot order) against the two launchers it stands for,
    including the shapes it hands back to them (more than 16 tokens, more than 512 experts)."""
    rng = np.random.default_rng(7 * E + T)
    scores = rng.uniform(0.05, 0.95, (T, E)).astype(np.float32) if mode == 0 else \
        hg.bf16_to_f32(hg.normal_bf16(E + T, (T, E)))
    biased = (scores + rng.normal(0, 0.05, (T, E))).astype(np.float32) if mode == 0 else scores
    scores[0, : E // 2] = scores[0, 0]          # a row with many exact ties: lower id wins
    if mode == 0:
        biased[0] = scores[0]
    cfg = L.make_config(64, 64, E, K, router_mode=mode, routed_scaling_factor=1.0 if mode else 2.5, n_shared_experts=0)
    slots = T * (K + 1)
    s_d, b_d = dev(scores), dev(biased)
    ids1, w1, o1 = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32), dev_empty(slots, np.int32)
    L.launch_moe_router_select(s_d, b_d, ids1, w1, cfg, T, None)
    L.launch_moe_slot_order(ids1, o1, slots, K, E, None, early)
    ids2, w2, o2 = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32), dev_empty(slots, np.int32)
    L.launch_moe_router_select_order(s_d, b_d, ids2, w2, o2, cfg, T, early, None)
    ids3, w3 = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32)
    L.launch_moe_router_select_order(s_d, b_d, ids3, w3, None, cfg, T, early, None)
    sync()
    assert np.array_equal(host(ids1), host(ids2)) and np.array_equal(host(ids1), host(ids3))
    assert np.array_equal(host(w1), host(w2)) and np.array_equal(host(w1), host(w3))
    assert np.array_equal(host(o1), host(o2))
    assert np.array_equal(np.sort(host(o2)), np.arange(slots))


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("E,H,T", [(96, 512, 16), (258, 1024, 37), (30, 4096, 64), (256, 6144, 19)])
def test_router_tiled_dots_are_bitwise_the_one_row_form(gpu, mode, E, H, T):
    """tests/cuda/glm_moe_test.cu moe_router_tiled_dots_are_bitwise_the_warp_form: from sixteen rows on the score rows
    come from the token-tiled kernel; scores, biased, ids and weights are bit for bit those of the one-row form."""
    K = 6
    x = hg.normal_bf16(mode + 11 + E, (T, H))
    gate = hg.normal_bf16(mode + 19 + H, (E, H), 1.0 / np.sqrt(H))
    bias = hg.normal_f32(mode + 5, (E,), 0.02)
    cfg = L.make_config(H, 64, E, K, router_mode=mode, routed_scaling_factor=1.0 if mode == 1 else 2.5)
    x_d, g_d, b_d = dev(x), dev(gate), (None if mode == 1 else dev(bias))
    from dgpp_amd import _lib
    res = []
    for tiled, tile in ((False, 0), (True, 0), (True, 2), (True, 4)):   # 0: the launcher's own choice for this batch
        ids_d, w_d = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32)
        sc_d, bi_d = dev_empty((T, E), np.float32), dev_empty((T, E), np.float32)
        sc_d.fill_(-7.0), bi_d.fill_(-7.0)
        _lib.load().dgpp_tune_set(10, tile)
        try:
            L.launch_moe_router(x_d, g_d, b_d, ids_d, w_d, sc_d, bi_d, cfg, T, None, None, tiled)
        finally:
            _lib.load().dgpp_tune_set(10, 0)
        sync()
        res.append([host(t).copy() for t in (sc_d, bi_d, ids_d, w_d)])
    for other in res[1:]:
        for a, b, name in zip(res[0], other, ("scores", "biased", "ids", "weights")):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), name
        assert not np.any(other[0] == -7.0), "every score of the batch is written"


@pytest.mark.parametrize("norm", [True, False])
@pytest.mark.parametrize("T,E,K,vocab", [(9, 40, 6, 17), (300, 256, 8, 1000), (1, 384, 16, 3)])
def test_hash_routes_bit_exact(gpu, norm, T, E, K, vocab):
    from test_oracle_moe import hash_route_case
    tokens, table, scores = hash_route_case(T, E, K, vocab, T + E)
    want_ids, want_w = np.empty((T, K), np.int32), np.empty((T, K), np.float32)
    orc.oracle().orc_hash_routes(orc.p(tokens), orc.p(table), orc.p(scores), T, vocab, E, K, 2.5, 1 if norm else 0,
                                 orc.p(want_ids), orc.p(want_w))
    cfg = L.make_config(64, 64, E, K, router_mode=0, routed_scaling_factor=2.5, norm_topk_prob=norm, n_shared_experts=0)
    ids_d, w_d = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32)
    import torch
    L.launch_moe_hash_routes(torch.from_numpy(tokens).to("cuda:0"), dev(table), dev(scores), ids_d, w_d, cfg, vocab, T)
    sync()
    assert np.array_equal(host(ids_d), want_ids)
    assert np.array_equal(host(w_d).view(np.uint32), want_w.view(np.uint32))
    soft = L.make_config(64, 64, E, K, router_mode=1, routed_scaling_factor=1.0, n_shared_experts=0)
    with pytest.raises(L.InvalidArgument):
        L.launch_moe_hash_routes(torch.from_numpy(tokens).to("cuda:0"), dev(table), dev(scores), ids_d, w_d, soft, vocab, T)
