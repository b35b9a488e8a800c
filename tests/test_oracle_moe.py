"""Pins the oracle's router and full-layer forward: against the compiled reference
(glm_moe_ref_router / glm_moe_ref_forward, src/models/glm/moe_reference.cpp:283-468) where
oracle/_ref exists, against the committed golden fixtures everywhere, and against closed forms."""
from pathlib import Path

import numpy as np
import pytest

import moe_data
import oracle_lib as orc
from dgpp_amd import hostgen as hg

GOLDEN = Path(__file__).resolve().parent / "golden"


def load_case(path):
    z = np.load(path)
    E, H, I, K, T, mode, seed = (int(v) for v in z["meta"])
    p = moe_data.make_problem(E, H, I, K, T, str(z["kind"]), seed, shared_kind=str(z["shared"]),
                              limit=float(z["limit"]), std=0.05)
    digest = np.array([m.payload.sum(dtype=np.uint64) for e in p.experts for m in e], np.uint64)
    assert np.array_equal(digest, z["digest"]), "the seeded weights no longer reproduce the fixture's"
    assert np.array_equal(p.x, z["x"]) and np.array_equal(p.router_gate, z["router_gate"])
    return p, mode, float(z["scaling"]), bool(z["norm"]), z


@pytest.mark.parametrize("path", sorted(GOLDEN.glob("moe_*.npz")), ids=lambda q: q.stem)
def test_golden_router_and_forward(path):
    p, mode, scaling, norm, z = load_case(path)
    ids, w, scores, biased = moe_data.orc_router(p, mode, scaling, norm)
    assert np.array_equal(ids, z["ids"])
    assert np.array_equal(w.view(np.uint32), z["weights"].view(np.uint32)), "router weights differ in bits"
    assert np.array_equal(biased, z["biased"])
    raw, bits = moe_data.orc_forward(p, ids, w)
    assert np.array_equal(bits, z["out"]), "layer output differs from the reference oracle's bits"
    # threads do not change any bit
    raw4, bits4 = moe_data.orc_forward(p, ids, w, threads=4)
    assert np.array_equal(raw, raw4) and np.array_equal(bits, bits4)


CASES = [
    (7, 128, 128, 3, 4, "fp8", "fp8", 0, 2.5, True, 10.0),
    (9, 128, 64, 4, 3, "nvfp4", "fp8", 0, 2.5, False, 10.0),
    (6, 64, 96, 2, 2, "nvfp4", "nvfp4", 2, 1.0, True, 3.0),
    (12, 128, 32, 8, 3, "mxfp4", "fp8", 1, 1.0, True, float("inf")),
    (5, 96, 64, 1, 2, "mxfp4", "fp8", 1, 1.0, True, 0.5),
]


@pytest.mark.parametrize("E,H,I,K,T,kind,shared,mode,scaling,norm,limit", CASES)
def test_live_reference_router_and_forward(E, H, I, K, T, kind, shared, mode, scaling, norm, limit):
    if orc.ref() is None:
        pytest.skip("oracle/_ref not built (no reference checkout)")
    p = moe_data.make_problem(E, H, I, K, T, kind, 100 + E + K, shared_kind=shared, limit=limit, std=0.05)
    rids, rw, rb = moe_data.ref_router(p, mode, scaling, norm)
    ids, w, scores, biased = moe_data.orc_router(p, mode, scaling, norm)
    assert np.array_equal(ids, rids) and np.array_equal(w.view(np.uint32), rw.view(np.uint32))
    assert np.array_equal(biased, rb)
    want = moe_data.ref_forward(p, mode, scaling, norm)
    raw, bits = moe_data.orc_forward(p, ids, w)
    assert np.array_equal(bits, want)


def test_live_reference_layer_handle_matches_the_one_shot_call():
    """The benchmark's CPU baseline keeps the reference oracle's weights between passes (ref_moe_layer_*): same
    output as the one-shot ref_moe_forward on an FP4 layer with an FP4 shared expert, repeated passes included."""
    r = orc.ref()
    if r is None or not hasattr(r, "ref_moe_layer_create"):
        pytest.skip("oracle/_ref not built (no reference checkout)")
    E, H, I, K, T = 6, 128, 64, 3, 4
    p = moe_data.make_problem(E, H, I, K, T, "mxfp4", 555, shared_kind="mxfp4", limit=float("inf"), std=0.05)
    want = moe_data.ref_forward(p, 1, 1.0, True)
    mats = [m for e in p.experts for m in e] + p.shared
    pay = np.ascontiguousarray(np.concatenate([m.payload.ravel() for m in mats]))
    sc = np.ascontiguousarray(np.concatenate([m.scales.ravel() for m in mats]))
    layer = r.ref_moe_layer_create(H, I, E, K, 1, 1.0, 1, p.limit, orc.p(p.router_gate), orc.p(p.router_bias), 32, orc.p(pay),
                                   pay.size, orc.p(sc), sc.size, None, 0)
    assert layer
    try:
        for _ in range(2):
            out = np.zeros((T, H), np.uint16)
            assert r.ref_moe_layer_forward(layer, orc.p(p.x), T, orc.p(out)) == 0
            assert np.array_equal(out, want)
    finally:
        r.ref_moe_layer_destroy(layer)


def test_router_tie_rule_all_equal_scores():
    """tests/cuda/glm_moe_test.cu:1498-1545: all-equal scores pick ids 0..K-1, weight s/(K*s)*scale."""
    E, K, T = 40, 8, 3
    scores = np.full((T, E), 0.5)
    ids = np.empty((T, K), np.int32)
    w = np.empty((T, K), np.float32)
    orc.oracle().orc_router_select(orc.p(scores), orc.p(scores), 0, T, E, K, 2.5, 1, orc.p(ids), orc.p(w))
    assert np.array_equal(ids, np.tile(np.arange(K, dtype=np.int32), (T, 1)))
    assert np.allclose(w, 0.5 / (K * 0.5) * 2.5, rtol=1e-7)
    # selection key and weight source are different rows: pick by biased, weigh by scores
    biased = scores.copy()
    biased[:, 30:38] += 1.0
    orc.oracle().orc_router_select(orc.p(scores), orc.p(biased), 0, T, E, K, 1.0, 0, orc.p(ids), orc.p(w))
    assert np.array_equal(ids[0], np.arange(30, 38)) and np.all(w == np.float32(0.5))


def test_router_select_brute_force():
    rng = np.random.default_rng(5)
    T, E, K = 16, 64, 6
    scores = rng.normal(size=(T, E))
    scores[:, 5] = scores[:, 9]          # exact ties: the lower id must win
    scores = hg.bf16_to_f32(hg.f32_to_bf16(scores.astype(np.float32))).astype(np.float64)
    ids = np.empty((T, K), np.int32)
    w = np.empty((T, K), np.float32)
    orc.oracle().orc_router_select(orc.p(scores), orc.p(scores), 1, T, E, K, 1.0, 1, orc.p(ids), orc.p(w))
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-scores[t, e], e))[:K]
        assert list(ids[t]) == sorted(order)
        pr = np.exp(scores[t] - scores[t].max())
        pr /= pr.sum()
        want = pr[ids[t]] / (pr[ids[t]].sum() + 1e-20)
        assert np.array_equal(w[t], hg.bf16_to_f32(hg.f32_to_bf16(want.astype(np.float32))))
        assert abs(w[t].sum() - 1) < 0.02


def test_swiglu_edges():
    """tests/cuda/glm_moe_test.cu:1547-1594 style edges, checked against the formula in fp64."""
    def bf(v):
        return hg.f32_to_bf16(np.array(v, np.float32))
    g = bf([0.0, 20.0, -20.0, 1.0, -1.0, 9.0, 100.0, 0.5])
    u = bf([1.0, 1.0, 1.0, 20.0, -20.0, -3.0, 2.0, 0.25])
    out = np.empty(8, np.uint16)
    orc.oracle().orc_swiglu(orc.p(g), orc.p(u), 8, 10.0, orc.p(out))
    gf, uf = hg.bf16_to_f32(g).astype(np.float64), hg.bf16_to_f32(u).astype(np.float64)
    gc = np.minimum(gf, 10.0)                       # gate: upper clamp only
    uc = np.clip(uf, -10.0, 10.0)
    silu = hg.bf16_to_f32(hg.f32_to_bf16((gc / (1 + np.exp(-gc))).astype(np.float32))).astype(np.float64)
    want = hg.f32_to_bf16((silu * uc).astype(np.float32))
    assert np.array_equal(out, want)
    assert hg.bf16_to_f32(out)[2] < 0 and abs(hg.bf16_to_f32(out)[2]) < 1e-6   # -20 is NOT clamped below
    assert hg.bf16_to_f32(out)[3] == hg.bf16_to_f32(bf([0.73046875 * 10.0]))[0]  # up clamped to +10


def test_forward_degenerate_reduces_to_one_expert():
    """top_k = 1, weight 1, no shared expert: the layer is one expert MLP; check against numpy fp64."""
    import np_ref
    p = moe_data.make_problem(3, 64, 32, 1, 2, "mxfp4", 21, shared_kind=None, limit=float("inf"), std=0.05)
    ids = np.array([[2], [0]], np.int32)
    w = np.ones((2, 1), np.float32)
    raw, bits = moe_data.orc_forward(p, ids, w)
    for t in range(2):
        g, u, d = p.experts[int(ids[t, 0])]
        x = np_ref.bf16_bits_to_f64(p.x[t])
        gd = np_ref.dequant_fp4(g.payload, g.scales, 32) @ x
        ud = np_ref.dequant_fp4(u.payload, u.scales, 32) @ x
        gb = np_ref.f32_to_bf16_f64(gd.astype(np.float32))
        ub = np_ref.f32_to_bf16_f64(ud.astype(np.float32))
        silu = np_ref.f32_to_bf16_f64((gb / (1 + np.exp(-gb))).astype(np.float32))
        act = np_ref.f32_to_bf16_f64((silu * ub).astype(np.float32))
        want = np_ref.dequant_fp4(d.payload, d.scales, 32) @ act
        assert np.allclose(raw[t], want, rtol=1e-12, atol=1e-300)


def hash_route_case(T, E, K, vocab, seed):
    rng = np.random.default_rng(seed)
    table = np.stack([np.sort(rng.permutation(E)[:K]) for _ in range(vocab)]).astype(np.int32)
    tokens = rng.integers(0, vocab, T).astype(np.int64)
    tokens[0], tokens[-1] = -5, vocab + 3                      # padding rows read table row 0
    scores = rng.uniform(0.01, 0.99, (T, E)).astype(np.float32)
    return tokens, table, scores


@pytest.mark.parametrize("norm", [1, 0])
def test_hash_routes_oracle_against_numpy(norm):
    """src/kernels/glm_moe.cu:917-949: the routes come from the table, the weights from the scores at those ids."""
    T, E, K, vocab = 9, 40, 6, 17
    tokens, table, scores = hash_route_case(T, E, K, vocab, 3)
    ids, w = np.empty((T, K), np.int32), np.empty((T, K), np.float32)
    orc.oracle().orc_hash_routes(orc.p(tokens), orc.p(table), orc.p(scores), T, vocab, E, K, 2.5, norm, orc.p(ids), orc.p(w))
    rows = np.where((tokens < 0) | (tokens >= vocab), 0, tokens)
    assert np.array_equal(ids, table[rows])
    sel = np.take_along_axis(scores, table[rows], axis=1)
    denom = np.zeros(T, np.float32)
    for j in range(K):                                          # the fp32 chain, one addition at a time
        denom = (denom + sel[:, j]).astype(np.float32)
    denom = (denom + np.float32(1e-20)).astype(np.float32)
    want = ((sel / denom[:, None]).astype(np.float32) * np.float32(2.5)).astype(np.float32) if norm else (sel * np.float32(2.5)).astype(np.float32)
    assert np.array_equal(w.view(np.uint32), want.view(np.uint32))
    if norm:
        assert np.allclose(w.sum(axis=1), 2.5, rtol=1e-6)
    # all-equal scores: every weight is 1 / K * scaling
    flat = np.full((T, E), 0.5, np.float32)
    orc.oracle().orc_hash_routes(orc.p(tokens), orc.p(table), orc.p(flat), T, vocab, E, K, 2.5, 1, orc.p(ids), orc.p(w))
    assert np.allclose(w, 2.5 / K, rtol=1e-6)
