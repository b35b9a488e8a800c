"""dgpp_minimax_router (src/kernels/minimax.hpp:56-60): FP32 gate, sigmoid scores, the bias in the ranking only,
FP32 weights. The reference's known answers; scores against the float64 oracle; ids and weights bit for bit the
oracle's selection run on the device's own scores (the selection is FP32 arithmetic with a fixed order)."""
import numpy as np
import pytest

import oracle_lib as orc
from dgpp_amd import hostgen as hg, launch as L
from gpu_util import dev, dev_empty, host, sync

pytestmark = pytest.mark.gpu


def run(x, gate, bias, topk, factor):
    rows, hidden = x.shape
    experts = gate.shape[0]
    xd, gd, bd = dev(x), dev(gate), dev(bias)
    scores = dev_empty((rows, experts), np.float32)
    ids = dev_empty((rows, topk), np.int32)
    w = dev_empty((rows, topk), np.float32)
    L.minimax_router(xd, gd, bd, rows, hidden, experts, topk, factor, scores, ids, w)
    sync()
    return host(scores), host(ids), host(w)


def test_reference_kernel_known_answer():
    # tests/cuda/minimax_test.cpp:667-675: FP32 router low bits decide an otherwise tied selection
    x = np.zeros((1, 128), np.uint16)
    x[0, 0] = hg.f32_to_bf16(np.array([1.0], np.float32))[0]
    gate = np.zeros((4, 128), np.float32)
    gate[:, 0] = [0.5001, 0.5002, -1, -2]
    _, ids, w = run(x, gate, np.zeros(4, np.float32), 1, 2.0)
    assert ids.tolist() == [[1]] and w.tolist() == [[2.0]]


def test_reference_unit_known_answer_and_tie_rule():
    # tests/unit/minimax_reference_test.cpp:56-61: zero logits, the bias selects, the unbiased scores normalise
    x = np.zeros((2, 64), np.uint16)
    gate = np.ones((4, 64), np.float32)
    scores, ids, w = run(x, gate, np.array([0, 10, 1, 0], np.float32), 2, 2.0)
    assert np.array_equal(scores, np.full((2, 4), 0.5, np.float32))
    assert ids.tolist() == [[1, 2]] * 2 and w.tolist() == [[1.0, 1.0]] * 2
    # all equal: the lower ids win
    _, ids, _ = run(np.zeros((1, 64), np.uint16), np.ones((9, 64), np.float32), np.zeros(9, np.float32), 4, 1.0)
    assert ids.tolist() == [[0, 1, 2, 3]]


@pytest.mark.parametrize("rows,hidden,experts,topk", [(64, 6144, 256, 8), (3, 100, 20, 5), (5, 1024, 700, 16), (1, 512, 4096, 8)])
def test_scores_against_the_oracle_and_selection_bit_for_bit(rows, hidden, experts, topk):
    print(f"minimax router rows={rows} hidden={hidden} experts={experts} topk={topk}", flush=True)
    rng = np.random.default_rng(rows * 31 + experts)
    x = hg.normal_bf16(500 + rows, (rows, hidden))
    gate = (rng.normal(0, 1.0, (experts, hidden)) / np.sqrt(hidden)).astype(np.float32)
    bias = rng.normal(0, 0.1, experts).astype(np.float32)
    scores, ids, w = run(x, gate, bias, topk, 2.5)
    want = np.empty((rows, experts), np.float64)
    orc.oracle().orc_minimax_router_scores(orc.p(x), orc.p(gate), rows, hidden, experts, orc.p(want))
    assert np.abs(scores.astype(np.float64) - want).max() <= 2e-6, "sigmoid scores"
    oid = np.empty((rows, topk), np.int32)
    ow = np.empty((rows, topk), np.float32)
    scores_c = np.ascontiguousarray(scores)
    orc.oracle().orc_minimax_route_scores(orc.p(scores_c), orc.p(bias), rows, experts, topk, 2.5, orc.p(oid), orc.p(ow))
    assert np.array_equal(ids, oid), "ids"
    assert np.array_equal(w.view(np.uint32), ow.view(np.uint32)), "weights are FP32, never narrowed, bit for bit"
    assert np.all(np.diff(ids, axis=1) > 0), "ascending ids"


def test_argument_rules():
    x = dev(np.zeros((1, 64), np.uint16))
    g = dev(np.zeros((4, 64), np.float32))
    b = dev(np.zeros(4, np.float32))
    s, i, w = dev_empty((1, 4), np.float32), dev_empty((1, 4), np.int32), dev_empty((1, 4), np.float32)
    L.minimax_router(x, g, b, 0, 64, 4, 2, 1.0, s, i, w)                # rows <= 0 returns at once
    for experts, topk in ((0, 1), (4, 0), (4, 17), (4, 5)):
        with pytest.raises(L.InvalidArgument):
            L.minimax_router(x, g, b, 1, 64, experts, topk, 1.0, s, i, w)
