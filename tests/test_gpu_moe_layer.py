"""The C++ host layer driver (the reference's GlmMoeLayer counterpart) end to end against the oracle,
at small shapes with every path (router from hidden rows, from given scores, given routes; decode
slots and grouped), plus the benchmark's layer shapes through size-independent properties."""
import ctypes as C

import numpy as np
import pytest
import torch

import moe_data
import oracle_lib as orc
from dgpp_amd import hostgen as hg, launch as L, moe_layer as ML
from gpu_util import DeviceMoe, dev, dev_empty, host, sync
from test_gpu_moe_slots import expert_budget

pytestmark = pytest.mark.gpu


def make_layer(p, d, mode, scaling, max_tokens):
    cfg = L.make_config(p.H, p.I, p.E, p.K, n_shared_experts=1 if p.shared else 0, routed_scaling_factor=scaling,
                        swiglu_limit=p.limit, router_mode=mode)
    views = list((L.MoeExpertView * (d.views.numel() // 96)).from_buffer_copy(bytes(host(d.views))))
    fmt = {"fp8": ML.EXPERTS_FP8, "nvfp4": ML.EXPERTS_NVFP4, "mxfp4": ML.EXPERTS_MXFP4}[p.kind]
    kw = {}
    if p.shared:
        if d.shared_view_base >= 0:
            kw = dict(shared_in_table=True, shared_inter=p.shared_I)
        else:
            kw = dict(shared_inter=p.shared_I, sh_payload=[t[0] for t in d.sh], sh_scales=[t[1] for t in d.sh])
    gate_d, bias_d = dev(p.router_gate), dev(p.router_bias)
    layer = ML.MoeLayer(cfg, fmt, views, max_tokens, router_gate=gate_d, router_bias=None if mode == 1 else bias_d, **kw)
    layer._keep2 = (gate_d, bias_d)
    return layer


CASES = [
    (16, 256, 128, 4, 3, "fp8", "fp8", 128, 0, 2.5, 10.0),
    (16, 512, 128, 4, 4, "nvfp4", "fp8", 256, 0, 2.5, 10.0),
    (10, 512, 64, 2, 2, "nvfp4", "nvfp4", 64, 2, 1.5, 10.0),
    (32, 1024, 256, 8, 8, "mxfp4", None, None, 1, 1.0, float("inf")),
    (24, 512, 128, 8, 1, "mxfp4", None, None, 1, 1.0, float("inf")),
    (16, 256, 128, 8, 6, "fp8", None, None, 1, 1.0, float("inf")),
]


@pytest.mark.parametrize("E,H,I,K,T,kind,shared,sI,mode,scaling,limit", CASES)
def test_layer_driver_vs_oracle(gpu, E, H, I, K, T, kind, shared, sI, mode, scaling, limit):
    p = moe_data.make_problem(E, H, I, K, T, kind, 500 + E + T, shared_kind=shared, shared_I=sI, limit=limit, std=0.05)
    d = DeviceMoe(p)
    layer = make_layer(p, d, mode, scaling, T)
    out = dev_empty((T, H), np.uint16)
    layer.enqueue_decode(d.x, H, out, T)
    sync()
    # read back the routes the layer used (device-to-device copy out of the layer's scratch)
    ids_t = torch.empty((T, K), dtype=torch.int32, device="cuda")
    w_t = torch.empty((T, K), dtype=torch.float32, device="cuda")
    hip = C.CDLL("libamdhip64.so")
    kDeviceToDevice = 3
    assert hip.hipMemcpy(C.c_void_p(ids_t.data_ptr()), C.c_void_p(layer.ids_ptr), T * K * 4, kDeviceToDevice) == 0
    assert hip.hipMemcpy(C.c_void_p(w_t.data_ptr()), C.c_void_p(layer.weights_ptr), T * K * 4, kDeviceToDevice) == 0
    sync()
    got_ids, got_w = host(ids_t), host(w_t)
    want_ids, want_w, _, biased = moe_data.orc_router(p, mode, scaling, True)
    if not np.array_equal(got_ids, want_ids):      # only near-ties may differ
        for t in range(T):
            a = list(set(got_ids[t]) ^ set(want_ids[t]))
            if a:
                gap = biased[t, a].max() - biased[t, a].min()
                assert gap <= (2.0 ** -7 * np.abs(biased[t, a]).max() if mode == 1 else 1e-5)
    # the expert path is judged on the routes the device chose
    raw, bits = moe_data.orc_forward(p, got_ids, got_w)
    expert_budget(host(out, np.uint16), raw, f"driver {kind}/{shared} T{T}")
    # given routes: decode and grouped paths agree bitwise with each other and with the full call
    out2 = dev_empty((T, H), np.uint16)
    layer.enqueue_decode_routed(d.x, H, ids_t, w_t, out2, T)
    sync()
    assert np.array_equal(host(out2), host(out))
    if not shared:
        out3 = dev_empty((T, H), np.uint16)
        layer.enqueue_grouped_routed(d.x, H, ids_t, w_t, out3, T)
        outf = dev_empty((T, H), np.float32)
        layer.enqueue_decode_routed(d.x, H, ids_t, w_t, None, T, out_f32=outf)
        sync()
        assert np.array_equal(host(out3), host(out))
        assert np.array_equal(hg.f32_to_bf16(host(outf)), host(out, np.uint16))
    with pytest.raises(L.InvalidArgument):
        layer.enqueue_decode(d.x, H, out, T + 1)
    layer.close()


def test_layer_from_given_scores_softmax(gpu):
    E, H, I, K, T = 64, 512, 128, 8, 4
    p = moe_data.make_problem(E, H, I, K, T, "mxfp4", 901, shared_kind=None, limit=float("inf"), std=0.05)
    d = DeviceMoe(p)
    layer = make_layer(p, d, 1, 1.0, T)
    logits = hg.bf16_to_f32(hg.normal_bf16(4242, (T, E)))       # router logits N(0,1), bf16 values
    out = dev_empty((T, H), np.uint16)
    lg = dev(logits)
    layer.enqueue_decode_scores(d.x, H, lg, lg, out, T)
    sync()
    l64 = logits.astype(np.float64)
    ids, w = np.empty((T, K), np.int32), np.empty((T, K), np.float32)
    orc.oracle().orc_router_select(orc.p(l64), orc.p(l64), 1, T, E, K, 1.0, 1, orc.p(ids), orc.p(w))
    raw, _ = moe_data.orc_forward(p, ids, w)
    expert_budget(host(out, np.uint16), raw, "scores-driven layer")
    # the selection as a launch of its own (bench switch 7) gives the same bits as the selection repeated in the
    # gate/up blocks
    out2 = dev_empty((T, H), np.uint16)
    from dgpp_amd import _lib
    _lib.load().dgpp_tune_set(7, 1)
    try:
        layer.enqueue_decode_scores(d.x, H, lg, lg, out2, T)
        sync()
    finally:
        _lib.load().dgpp_tune_set(7, 0)
    assert np.array_equal(host(out2, np.uint16), host(out, np.uint16))
    layer.close()


@pytest.mark.parametrize("E,H,I,K,T,kind,shared,sI", [(16, 512, 128, 4, 4, "nvfp4", "fp8", 256), (16, 256, 128, 4, 3, "fp8", "fp8", 128),
                                                      (10, 512, 64, 2, 2, "nvfp4", "nvfp4", 64), (12, 512, 128, 8, 24, "mxfp4", "fp8", 128)])
def test_shared_expert_passes_beside_the_routed_ones_give_the_same_bits(gpu, E, H, I, K, T, kind, shared, sI):
    """The layer driver runs the shared expert's gate/up and down passes on a second stream beside the routed passes
    (forked and joined with events). Same bits as with everything on the caller's stream (bench switch 9), eagerly on
    a side stream of the caller and as a captured graph replayed several times with eager work in between."""
    from dgpp_amd import _lib
    p = moe_data.make_problem(E, H, I, K, T, kind, 700 + E + T, shared_kind=shared, shared_I=sI, limit=10.0, std=0.05)
    d = DeviceMoe(p)
    layer = make_layer(p, d, 0, 2.5, T)
    want = dev_empty((T, H), np.uint16)
    _lib.load().dgpp_tune_set(9, 3)           # one stream, the accumulation a launch of its own
    try:
        layer.enqueue_decode(d.x, H, want, T)
        sync()
        want_h = host(want, np.uint16).copy()
        _lib.load().dgpp_tune_set(9, 4)       # one stream, the accumulation folded into the shared down pass
        want.zero_()
        layer.enqueue_decode(d.x, H, want, T)
        sync()
        assert np.array_equal(host(want, np.uint16), want_h), "folded accumulation"
    finally:
        _lib.load().dgpp_tune_set(9, 0)
    ids, w, _, _ = moe_data.orc_router(p, 0, 2.5, True)
    raw, _ = moe_data.orc_forward(p, ids, w)
    expert_budget(want_h, raw, "shared-expert layer on one stream")
    s = torch.cuda.Stream()
    got = dev_empty((T, H), np.uint16)
    _lib.load().dgpp_tune_set(9, 2)           # the two-stream form at every batch size (default: from three tokens on)
    try:
        _two_stream_runs(layer, d, got, want_h, T, H, s)
    finally:
        _lib.load().dgpp_tune_set(9, 0)
    layer.close()


def _two_stream_runs(layer, d, got, want_h, T, H, s):
    with torch.cuda.stream(s):
        for _ in range(3):
            got.zero_()
            layer.enqueue_decode(d.x, H, got, T, s)
            s.synchronize()
            assert np.array_equal(host(got, np.uint16), want_h), "eager, passes on two streams"
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            layer.enqueue_decode(d.x, H, got, T, s)
            layer.enqueue_decode(d.x, H, got, T, s)
        for _ in range(3):
            got.zero_()                       # eager work between the replays
            s.synchronize()
            g.replay()
            s.synchronize()
            assert np.array_equal(host(got, np.uint16), want_h), "graph replay"


GOLDEN_CASES = sorted((__import__("pathlib").Path(__file__).resolve().parent / "golden").glob("moe_*.npz"))


@pytest.mark.parametrize("path", GOLDEN_CASES, ids=lambda q: q.stem)
def test_layer_driver_vs_reference_golden_fixtures(gpu, path):
    """The committed fixtures hold what the REFERENCE's own CPU oracle (glm_moe_ref_router / glm_moe_ref_forward, compiled
    from its sources) produced for four seeded layers. The HIP path meets them directly here: the layer driver's routed
    ids equal the fixture's (a difference must be a certified near-tie of the fixture's biased scores), and its BF16
    output is held to the reference's expert budget (hard 12 ulps, soft 4 ulps on < 2 %, l2 < 4e-3, floor 2 % of the
    RMS; tests/cuda/glm_moe_test.cu:606-658) against the fixture's output bits."""
    from test_oracle_moe import load_case
    p, mode, scaling, norm, z = load_case(path)
    assert norm, "the fixtures use renormalised top-k weights (the layer configuration's default)"
    T, K, H = p.T, p.K, p.H
    d = DeviceMoe(p)
    layer = make_layer(p, d, mode, scaling, T)
    out = dev_empty((T, H), np.uint16)
    layer.enqueue_decode(d.x, H, out, T)
    sync()
    ids_t = torch.empty((T, K), dtype=torch.int32, device="cuda")
    hip = C.CDLL("libamdhip64.so")
    assert hip.hipMemcpy(C.c_void_p(ids_t.data_ptr()), C.c_void_p(layer.ids_ptr), T * K * 4, 3) == 0
    sync()
    got_ids, want_ids, biased = host(ids_t), z["ids"], z["biased"]
    same_routes = np.array_equal(got_ids, want_ids)
    if not same_routes:
        for t in range(T):
            a = list(set(got_ids[t]) ^ set(want_ids[t]))
            if a:
                gap = biased[t, a].max() - biased[t, a].min()
                assert gap <= (2.0 ** -7 * np.abs(biased[t, a]).max() if mode == 1 else 1e-5), "routes differ beyond a near-tie"
        pytest.skip("a near-tie routed differently: the fixture's output belongs to other experts")
    got = host(out, np.uint16)
    strict = hg.bf16_to_f32(z["out"]).astype(np.float64)
    rms = float(np.sqrt(np.mean(strict ** 2)))
    floor_frac = 0.02 * rms / max(np.abs(strict).max(), 1e-30)
    hard = orc.compare_bf16(got, strict, 12.0, floor_frac)
    soft = orc.compare_bf16(got, strict, 4.0, floor_frac)
    assert hard.mismatches == 0 and hard.nan_pattern_errors == 0, f"{path.stem}: hard budget, max {hard.max_ulps:.1f} ulps"
    assert soft.mismatches < 0.02 * soft.total, f"{path.stem}: soft budget {soft.mismatches}/{soft.total}"
    assert hard.l2_rel < 4e-3, f"{path.stem}: l2 {hard.l2_rel}"
    layer.close()
