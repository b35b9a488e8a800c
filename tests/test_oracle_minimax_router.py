"""Pins the oracle's MiniMax routing (orc_minimax_route_scores, orc_minimax_router_scores): the reference's own
known answers (tests/unit/minimax_reference_test.cpp:56-61, tests/cuda/minimax_test.cpp:667-675), the compiled
reference statement (src/models/minimax/reference.cpp:96-113) bit for bit where it was built, a numpy brute force,
and the tie rule."""
import numpy as np
import pytest

import oracle_lib as orc
from dgpp_amd import hostgen as hg


def route(scores, bias, topk, factor):
    scores = np.ascontiguousarray(scores, np.float32)
    bias = np.ascontiguousarray(bias, np.float32)
    rows, experts = scores.shape
    ids = np.empty((rows, topk), np.int32)
    w = np.empty((rows, topk), np.float32)
    orc.oracle().orc_minimax_route_scores(orc.p(scores), orc.p(bias), rows, experts, topk, factor, orc.p(ids), orc.p(w))
    return ids, w


def test_reference_unit_known_answer():
    # logits 0 -> every score 0.5; the bias picks experts 1 and 2; the unbiased scores normalise: 0.5 / 1.0 * 2
    ids, w = route(np.full((1, 4), 0.5, np.float32), np.array([0, 10, 1, 0], np.float32), 2, 2.0)
    assert ids.tolist() == [[1, 2]] and w.tolist() == [[1.0, 1.0]]


def test_reference_kernel_known_answer_keeps_fp32_low_bits():
    logits = np.array([[0.5001, 0.5002, -1.0, -2.0]], np.float32)
    scores = (1.0 / (1.0 + np.exp(-logits.astype(np.float64)))).astype(np.float32)
    ids, w = route(scores, np.zeros(4, np.float32), 1, 2.0)
    assert ids.tolist() == [[1]] and w.tolist() == [[2.0]]


def test_ties_go_to_the_lower_id_and_ids_come_back_ascending():
    ids, w = route(np.full((2, 9), 0.25, np.float32), np.zeros(9, np.float32), 4, 1.0)
    assert ids.tolist() == [[0, 1, 2, 3]] * 2
    assert np.array_equal(w, np.full((2, 4), np.float32(0.25) / np.float32(1.0), np.float32))
    bias = np.array([0, 0, 5, 0, 0, 5, 0, 0, 0], np.float32)
    ids, _ = route(np.full((1, 9), 0.25, np.float32), bias, 3, 1.0)
    assert ids.tolist() == [[0, 2, 5]]


def test_against_numpy_brute_force():
    rng = np.random.default_rng(5)
    rows, experts, topk, factor = 7, 96, 6, np.float32(2.5)
    scores = rng.random((rows, experts), dtype=np.float32)
    bias = rng.normal(0, 0.3, experts).astype(np.float32)
    ids, w = route(scores, bias, topk, float(factor))
    for r in range(rows):
        key = scores[r] + bias          # float32 adds
        order = sorted(range(experts), key=lambda e: (-key[e], e))
        picked = sorted(order[:topk])
        assert ids[r].tolist() == picked
        s = np.float32(0)
        for e in picked:
            s = np.float32(s + scores[r, e])
        want = [np.float32(np.float32(scores[r, e] / max(s, np.float32(1e-20))) * factor) for e in picked]
        assert np.array_equal(w[r], np.array(want, np.float32))


@pytest.mark.skipif(orc.ref() is None, reason="the compiled reference (oracle/_ref) is not built here")
def test_bit_for_bit_the_compiled_reference_statement():
    rng = np.random.default_rng(9)
    experts, topk = 64, 8
    for trial in range(20):
        logits = rng.normal(0, 2, experts).astype(np.float32)
        if trial % 4 == 0:
            logits[: experts // 2] = logits[0]          # exact ties
        bias = rng.normal(0, 0.2, experts).astype(np.float32)
        rid = np.empty(topk, np.int32)
        rw = np.empty(topk, np.float32)
        assert orc.ref().ref_minimax_route(orc.p(logits), orc.p(bias), experts, topk, 2.0, orc.p(rid), orc.p(rw)) == 0
        scores = (np.float32(1.0) / (np.float32(1.0) + np.exp(-logits, dtype=np.float32))).astype(np.float32)
        ids, w = route(scores[None, :], bias, topk, 2.0)
        assert np.array_equal(ids[0], rid)
        # the reference forms its sigmoid with the C library's float exp; numpy's may differ in the last bit
        assert np.allclose(w[0], rw, rtol=3e-7, atol=0)
    bad = np.empty(1, np.int32)
    badw = np.empty(1, np.float32)
    z = np.zeros(4, np.float32)
    assert orc.ref().ref_minimax_route(orc.p(z), orc.p(z), 4, 5, 1.0, orc.p(bad), orc.p(badw)) == 1   # topk > experts throws


def test_scores_are_the_sigmoid_of_the_float64_dot():
    rng = np.random.default_rng(2)
    rows, hidden, experts = 3, 40, 5
    x = hg.normal_bf16(77, (rows, hidden))
    gate = rng.normal(0, 0.2, (experts, hidden)).astype(np.float32)
    got = np.empty((rows, experts), np.float64)
    orc.oracle().orc_minimax_router_scores(orc.p(x), orc.p(gate), rows, hidden, experts, orc.p(got))
    want = 1.0 / (1.0 + np.exp(-(hg.bf16_to_f32(x).astype(np.float64) @ gate.astype(np.float64).T)))
    assert np.allclose(got, want, rtol=1e-13, atol=0)
