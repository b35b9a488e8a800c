"""The routed expert chain of a small decode batch in ONE launch (dgpp_launch_moe_slot_chain*): bit for bit the
launches it stands for (launch_moe_slot_gate_up_swiglu*, then launch_moe_slot_down_accum*), readiness words back
at rest after every launch, and the bounded wait's give-up path forced from the host.
"""
import numpy as np
import pytest
import torch

import moe_data
from dgpp_amd import _lib, launch as L
from gpu_util import DeviceMoe, dev, dev_empty, host, sync

pytestmark = pytest.mark.gpu

CASES = [
    # E, H, I, K, T, kind
    (32, 1024, 256, 8, 1, "mxfp4"),
    (32, 1024, 256, 8, 2, "mxfp4"),
    (32, 1024, 256, 8, 8, "mxfp4"),
    (12, 256, 64, 8, 12, "mxfp4"),      # sharers of an expert in both ballot words
    (64, 4096, 1024, 8, 4, "mxfp4"),    # the headline layer's row widths
    (16, 1024, 256, 8, 2, "nvfp4"),
    (16, 2048, 512, 6, 5, "nvfp4"),     # six waves of eight carry a slot each
    (10, 512, 64, 2, 3, "nvfp4"),       # top_k 2: the four-wave block
    (12, 384, 96, 3, 3, "fp8"),
    (24, 512, 128, 8, 16, "fp8"),
]


def routes(p, K, T, seed):
    rng = np.random.default_rng(seed)
    ids = np.stack([np.sort(rng.choice(p.E, K, replace=False)) for _ in range(T)]).astype(np.int32)
    w = rng.random((T, K), dtype=np.float32) + 0.05
    w = (w / w.sum(1, keepdims=True)).astype(np.float32)
    return ids, w


def two_launches(p, d, ids_d, w_d, T, K, f32):
    slots = T * (K + 1)
    act = dev_empty((slots, p.I), np.uint16)
    act.zero_()
    out = dev_empty((T, p.H), np.float32 if f32 else np.uint16)
    if p.kind == "fp8":
        L.launch_moe_slot_gate_up_swiglu(d.x, p.H, ids_d, None, d.views, p.I, p.H, 0, 0, None, None, None, None, act, p.I,
                                         slots, K, p.limit, None)
        L.launch_moe_slot_down_accum(act, p.I, ids_d, d.views, p.H, p.I, T, K, w_d, None if f32 else out, out if f32 else None)
    else:
        L.launch_moe_slot_gate_up_swiglu_fp4(d.x, p.H, ids_d, None, d.views, p.I, p.H, 0, 0, None, None, None, None, act,
                                             p.I, slots, K, p.limit, None, -1, d.fp4_group)
        L.launch_moe_slot_down_accum_fp4(act, p.I, ids_d, d.views, p.H, p.I, T, K, w_d, None if f32 else out,
                                         out if f32 else None, None, d.fp4_group)
    sync()
    return host(act, np.uint16), host(out, None if f32 else np.uint16)


def one_launch(p, d, ids_d, w_d, T, K, f32, ready, status, spins=0):
    slots = T * (K + 1)
    act = dev_empty((slots, p.I), np.uint16)
    act.zero_()
    out = dev_empty((T, p.H), np.float32 if f32 else np.uint16)
    out.zero_()
    if p.kind == "fp8":
        L.launch_moe_slot_chain(d.x, p.H, ids_d, d.views, p.I, p.H, act, p.I, T, K, p.limit, w_d, None if f32 else out,
                                out if f32 else None, ready, status, spins)
    else:
        L.launch_moe_slot_chain_fp4(d.x, p.H, ids_d, d.views, p.I, p.H, act, p.I, T, K, p.limit, w_d, None if f32 else out,
                                    out if f32 else None, ready, status, spins, None, d.fp4_group)
    sync()
    return host(act, np.uint16), host(out, None if f32 else np.uint16)


def routed_rows(act, T, K):
    return np.stack([act[t * (K + 1) + j] for t in range(T) for j in range(K)])


@pytest.mark.parametrize("E,H,I,K,T,kind", CASES)
def test_chain_is_bitwise_the_two_launches(E, H, I, K, T, kind):
    print(f"chain case E={E} H={H} I={I} K={K} T={T} {kind}", flush=True)
    p = moe_data.make_problem(E, H, I, K, T, kind, 9100 + T, shared_kind=None, limit=float("inf") if kind != "fp8" else 9.0,
                              std=0.05)
    d = DeviceMoe(p)
    ids, w = routes(p, K, T, 77 + T)
    ids_d, w_d = dev(ids), dev(w)
    nbytes = L.moe_slot_chain_ready_bytes(T, K)
    assert nbytes == T * K * 128
    ready = torch.zeros(nbytes // 4, dtype=torch.int32, device="cuda:0")
    status = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    for f32 in (False, True):
        act2, out2 = two_launches(p, d, ids_d, w_d, T, K, f32)
        # twice in a row on the same readiness words: they are back at rest after every launch
        for rep in range(2):
            act1, out1 = one_launch(p, d, ids_d, w_d, T, K, f32, ready, status)
            assert int(status.item()) == 0, "a bounded wait gave up"
            assert not host(ready).any(), "readiness words not back at zero"
            assert np.array_equal(routed_rows(act1, T, K), routed_rows(act2, T, K)), f"act rows differ (rep {rep})"
            assert np.array_equal(out1.view(np.uint32 if f32 else np.uint16), out2.view(np.uint32 if f32 else np.uint16)), \
                f"outputs differ (f32={f32}, rep {rep})"


def test_chain_falls_back_outside_its_form():
    """No readiness words, or more routed slots than the form takes: the launcher runs the two launches, same bits."""
    E, H, I, K, T = 16, 512, 128, 4, 3
    p = moe_data.make_problem(E, H, I, K, T, "mxfp4", 9300, shared_kind=None, limit=float("inf"), std=0.05)
    d = DeviceMoe(p)
    ids, w = routes(p, K, T, 5)
    ids_d, w_d = dev(ids), dev(w)
    act2, out2 = two_launches(p, d, ids_d, w_d, T, K, False)
    act1, out1 = one_launch(p, d, ids_d, w_d, T, K, False, None, None)
    assert np.array_equal(routed_rows(act1, T, K), routed_rows(act2, T, K)) and np.array_equal(out1, out2)
    lib = _lib.load()
    lib.dgpp_tune_set(12, 1)
    try:
        ready = torch.zeros(L.moe_slot_chain_ready_bytes(T, K) // 4, dtype=torch.int32, device="cuda:0")
        status = torch.zeros(1, dtype=torch.int32, device="cuda:0")
        act1, out1 = one_launch(p, d, ids_d, w_d, T, K, False, ready, status)
    finally:
        lib.dgpp_tune_set(12, 0)
    assert np.array_equal(out1, out2)


def test_chain_wait_gives_up_and_reports():
    """The give-up path, forced from the host: readiness words that were NOT zeroed (set to the wrap value, so the
    producers' count can never reach what the readers wait for) and a spin limit of four polls. Every wavefront still
    exits; the status word is raised; after the words are zeroed again the next launch is right."""
    E, H, I, K, T = 32, 1024, 256, 8, 4
    p = moe_data.make_problem(E, H, I, K, T, "mxfp4", 9400, shared_kind=None, limit=float("inf"), std=0.05)
    d = DeviceMoe(p)
    ids, w = routes(p, K, T, 11)
    ids_d, w_d = dev(ids), dev(w)
    _, out2 = two_launches(p, d, ids_d, w_d, T, K, False)
    words = L.moe_slot_chain_ready_bytes(T, K) // 4
    ready = torch.full((words,), 0x7FFFFFF0, dtype=torch.int32, device="cuda:0")   # above any wrap value: the first count wraps
    status = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    one_launch(p, d, ids_d, w_d, T, K, False, ready, status, spins=4)
    assert int(status.item()) == 1, "the readers should have given up"
    ready.zero_()
    status.zero_()
    _, out1 = one_launch(p, d, ids_d, w_d, T, K, False, ready, status)
    assert int(status.item()) == 0 and not host(ready).any()
    assert np.array_equal(out1, out2)


def test_layer_driver_takes_the_chain_and_matches_the_two_launch_form():
    from test_gpu_moe_layer import make_layer
    E, H, I, K, T = 32, 1024, 256, 8, 4
    p = moe_data.make_problem(E, H, I, K, T, "mxfp4", 9500, shared_kind=None, limit=float("inf"), std=0.05)
    d = DeviceMoe(p)
    lib = _lib.load()
    outs = []
    for knob in (2, 0):     # 2: the driver takes the one-launch chain; 0: its default, the launches the chain stands for
        lib.dgpp_tune_set(12, knob)
        try:
            layer = make_layer(p, d, L.ROUTER_SOFTMAX_TOPK, 1.0, T)
            out = dev_empty((T, H), np.uint16)
            for _ in range(2):
                layer.enqueue_decode(d.x, H, out, T)
            layer.check()
            outs.append(host(out, np.uint16).copy())
            layer.close()
        finally:
            lib.dgpp_tune_set(12, 0)
    assert np.array_equal(outs[0], outs[1])


def test_chain_replays_in_a_graph():
    """Captured once, replayed with eager work between the replays: every replay equals the eager result."""
    E, H, I, K, T = 32, 1024, 256, 8, 8
    p = moe_data.make_problem(E, H, I, K, T, "mxfp4", 9600, shared_kind=None, limit=float("inf"), std=0.05)
    d = DeviceMoe(p)
    ids, w = routes(p, K, T, 3)
    ids_d, w_d = dev(ids), dev(w)
    _, want = two_launches(p, d, ids_d, w_d, T, K, False)
    ready = torch.zeros(L.moe_slot_chain_ready_bytes(T, K) // 4, dtype=torch.int32, device="cuda:0")
    status = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    slots = T * (K + 1)
    act = dev_empty((slots, I), np.uint16)
    out = dev_empty((T, H), np.uint16)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        L.launch_moe_slot_chain_fp4(d.x, H, ids_d, d.views, I, H, act, I, T, K, p.limit, w_d, out, None, ready, status, 0,
                                    stream, d.fp4_group)
        stream.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            L.launch_moe_slot_chain_fp4(d.x, H, ids_d, d.views, I, H, act, I, T, K, p.limit, w_d, out, None, ready, status,
                                        0, stream, d.fp4_group)
        for rep in range(4):
            out.zero_()
            g.replay()
            stream.synchronize()
            assert np.array_equal(host(out, np.uint16), want), f"replay {rep} differs"
            assert int(status.item()) == 0 and not host(ready).any()
            scratch = torch.ones(1 << 16, device="cuda:0")   # eager work of the program's own between replays
            scratch.add_(1.0)
    sync()


@pytest.mark.parametrize("kind,mode,E,H,I,K,T", [
    ("mxfp4", 1, 64, 1024, 256, 8, 1),
    ("mxfp4", 1, 256, 4096, 1024, 8, 1),     # the headline layer's one-token step
    ("nvfp4", 0, 96, 2048, 512, 6, 1),
    ("fp8", 0, 48, 512, 128, 4, 1),
    ("mxfp4", 1, 64, 1024, 256, 8, 3),       # more than one token: selection first, then the chain
    ("mxfp4", 1, 640, 1024, 256, 8, 1),      # more experts than the in-launch selection takes
])
def test_select_chain_is_bitwise_select_then_the_launches(kind, mode, E, H, I, K, T):
    """Selection inside the one-launch chain (one token) against launch_moe_router_select + gate/up + down/accumulate:
    the same ids, weights, act rows and output rows, also for the calls it hands on (several tokens, many experts)."""
    from dgpp_amd import hostgen as hg
    print(f"select chain case {kind} mode={mode} E={E} H={H} I={I} K={K} T={T}", flush=True)
    p = moe_data.make_problem(E, H, I, K, T, kind, 9700 + E + T, shared_kind=None, limit=7.0, std=0.05)
    d = DeviceMoe(p)
    rng = np.random.default_rng(13 * E + T)
    scores = rng.uniform(0.05, 0.95, (T, E)).astype(np.float32) if mode == 0 else hg.bf16_to_f32(hg.normal_bf16(E + T, (T, E)))
    biased = (scores + rng.normal(0, 0.05, (T, E))).astype(np.float32) if mode == 0 else scores
    cfg = L.make_config(H, I, E, K, router_mode=mode, routed_scaling_factor=1.0 if mode else 2.5, n_shared_experts=0)
    s_d, b_d = dev(scores), dev(biased)
    ids1, w1 = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32)
    ids2, w2 = dev_empty((T, K), np.int32), dev_empty((T, K), np.float32)
    L.launch_moe_router_select(s_d, b_d, ids1, w1, cfg, T, None)
    act_a, out_a = two_launches(p, d, ids1, w1, T, K, False)
    ready = torch.zeros(L.moe_slot_chain_ready_bytes(T, K) // 4, dtype=torch.int32, device="cuda:0")
    status = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    slots = T * (K + 1)
    for rep in range(2):
        act = dev_empty((slots, I), np.uint16)
        act.zero_()
        out = dev_empty((T, H), np.uint16)
        out.zero_()
        if kind == "fp8":
            L.launch_moe_select_slot_chain(s_d, b_d, ids2, w2, cfg, T, d.x, H, d.views, I, H, act, I, p.limit, out, None, ready,
                                           status)
        else:
            L.launch_moe_select_slot_chain_fp4(s_d, b_d, ids2, w2, cfg, T, d.x, H, d.views, I, H, act, I, p.limit, out, None,
                                               ready, status, 0, None, d.fp4_group)
        sync()
        assert int(status.item()) == 0 and not host(ready).any()
        assert np.array_equal(host(ids1), host(ids2)), "ids"
        assert np.array_equal(host(w1).view(np.uint32), host(w2).view(np.uint32)), "weights"
        assert np.array_equal(routed_rows(host(act, np.uint16), T, K), routed_rows(act_a, T, K)), "act rows"
        assert np.array_equal(host(out, np.uint16), out_a), f"output rows (rep {rep})"


def test_layer_driver_one_token_step_is_one_launch_with_the_same_bits():
    from test_gpu_moe_layer import make_layer
    E, H, I, K, T = 64, 1024, 256, 8, 1
    p = moe_data.make_problem(E, H, I, K, T, "mxfp4", 9800, shared_kind=None, limit=float("inf"), std=0.05)
    d = DeviceMoe(p)
    lib = _lib.load()
    outs = []
    for knob in (2, 0):     # 2: the driver takes the one-launch chain; 0: its default, the launches the chain stands for
        lib.dgpp_tune_set(12, knob)
        try:
            layer = make_layer(p, d, L.ROUTER_SOFTMAX_TOPK, 1.0, T)
            out = dev_empty((T, H), np.uint16)
            for _ in range(2):
                layer.enqueue_decode(d.x, H, out, T)
            layer.check()
            outs.append(host(out, np.uint16).copy())
            layer.close()
        finally:
            lib.dgpp_tune_set(12, 0)
    assert np.array_equal(outs[0], outs[1])
