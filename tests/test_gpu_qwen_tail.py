"""The gated shared expert's decode tail with block-FP8 weights (src/kernels/qwen_moe.hpp:18-87): bitwise the
unfused chain of launchers it stands for, the shared gate in the reference's summation order, and the whole
tail against the CPU oracle with the reference comparator of a GEMV stage."""
import numpy as np
import pytest

import mxfp8_data as md
import oracle_lib as orc
from dgpp_amd import hostgen as hg, launch as L
from gpu_util import dev, dev_empty, host, sync
from np_ref import bf16_bits_to_f64

pytestmark = pytest.mark.gpu


def f32(a):
    return np.asarray(a, dtype=np.float32)


def gate_in_kernel_order(x, stride, g, tokens, hidden):
    """The shared gate exactly as the kernel sums it: 32 strided lanes over 16-byte vectors, low element of a
    word before the high one, each step one fused multiply-add, then the xor tree 16, 8, 4, 2, 1."""
    xs = bf16_bits_to_f64(x.reshape(tokens, stride)[:, :hidden])
    gs = bf16_bits_to_f64(g)
    vecs = hidden // 8
    dot = np.zeros((tokens, 32), dtype=np.float32)
    for v0 in range(0, vecs, 32):
        lanes = np.arange(32) + v0
        live = lanes < vecs
        for e in range(8):
            k = np.where(live, lanes * 8 + e, 0)
            term = np.where(live, xs[:, k] * gs[k][None, :], 0.0)        # bf16 * bf16: exact in float64
            dot = np.where(live, (term + dot.astype(np.float64)).astype(np.float32), dot)
    for off in (16, 8, 4, 2, 1):
        dot = (dot + dot[:, np.arange(32) ^ off]).astype(np.float32)
    return dot[:, 0]


@pytest.mark.parametrize("tokens,hidden,stride", [(1, 2048, 2048), (8, 4096, 4096), (13, 264, 264), (3, 8, 8)])
def test_shared_gate(gpu, tokens, hidden, stride):
    x = hg.normal_bf16(0x51A0 + hidden, (tokens, stride), 1.0)
    g = hg.normal_bf16(0x51A1 + hidden, (hidden,), 0.05)
    w = dev_empty((tokens,), np.float32)
    L.qwen_moe_shared_gate_bf16(dev(x), dev(g), w, tokens, hidden)
    sync()
    got = host(w)
    logit = md.f32_to_bf16_bits(gate_in_kernel_order(x, stride, g, tokens, hidden))
    lg = bf16_bits_to_f64(logit)
    want = bf16_bits_to_f64(md.f32_to_bf16_bits(f32(1.0 / (1.0 + np.exp(-lg)))))
    assert np.array_equal(got.astype(np.float64), want)
    # and the oracle's double dot: the same weight unless the two logits straddle a BF16 rounding boundary
    ow = np.empty(tokens, dtype=np.float32)
    orc.oracle().orc_shared_gate(orc.p(x), stride, orc.p(g), tokens, hidden, orc.p(ow))
    assert np.all(np.abs(got - ow) <= 2.0 ** -7 * np.abs(ow))
    none = dev_empty((tokens,), np.float32)
    L.qwen_moe_shared_gate_bf16(dev(x), None, none, tokens, hidden)
    sync()
    assert np.all(host(none) == 1.0)


def make_tail(tokens, H, S, rs, cs, seed, top_k):
    x = hg.normal_bf16(seed, (tokens, H), 1.0)
    g = hg.normal_bf16(seed + 1, (H,), 0.03)
    mats = []
    for i, (r, c) in enumerate(((S, H), (S, H), (H, S))):
        wt = hg.f32_to_bf16(hg.normal_f32(seed + 2 + i, (r, c), 0.03))
        mats.append(hg.encode_fp8_blocks(wt, 1 << rs, 1 << cs))
    acc = hg.normal_f32(seed + 5, (tokens, H), 0.3)
    contrib = hg.normal_f32(seed + 6, (tokens * (top_k + 1), H), 0.3)
    weights = np.abs(hg.normal_f32(seed + 7, (tokens, top_k), 0.2)).astype(np.float32)
    return x, g, mats, acc, contrib, weights


CASES = [(1, 2048, 512, 7, 7, 8), (4, 1024, 768, 7, 7, 8), (8, 2048, 256, 7, 7, 10), (5, 512, 1024, 0, 5, 16),
         (2, 96, 48, 7, 7, 1), (7, 4096, 512, 7, 7, 8)]


@pytest.mark.parametrize("tokens,H,S,rs,cs,top_k", CASES)
def test_tail_is_bitwise_the_unfused_chain_and_meets_the_oracle(gpu, tokens, H, S, rs, cs, top_k):
    x, g, mats, acc, contrib, weights = make_tail(tokens, H, S, rs, cs, 0x7A11 + H + S + tokens, top_k)
    x_d, g_d = dev(x), dev(g)
    (gp, gs), (up, us), (dp, ds) = [(dev(p), dev(s)) for p, s in mats]
    acc_d, contrib_d, weights_d = dev(acc), dev(contrib), dev(weights)

    # the unfused chain
    gate_o, up_o, act_o = (dev_empty((tokens, S), np.uint16) for _ in range(3))
    L.launch_scale_gemm_grid_bf16(x_d, H, gp, gs, gate_o, tokens, S, H, None, 0, rs, cs)
    L.launch_scale_gemm_grid_bf16(x_d, H, up, us, up_o, tokens, S, H, None, 0, rs, cs)
    L.launch_moe_swiglu_clamp(gate_o, up_o, act_o, tokens * S, float("inf"))
    down_o = dev_empty((tokens, H), np.float32)
    L.launch_scale_gemm_grid_f32(act_o, S, dp, ds, down_o, tokens, H, S, None, 0, rs, cs)
    sw_o = dev_empty((tokens,), np.float32)
    L.qwen_moe_shared_gate_bf16(x_d, g_d, sw_o, tokens, H)
    rows = dev(np.arange(tokens, dtype=np.int32))
    sum_o = acc_d.clone()
    L.launch_moe_accum(sum_o, down_o, rows, sw_o, tokens, H)
    out_o = dev_empty((tokens, H), np.uint16)
    L.launch_moe_round_bf16(out_o, sum_o, tokens * H)
    routed_o = dev_empty((tokens, H), np.float32)
    L.launch_moe_slot_accum_routed_f32(routed_o, contrib_d, weights_d, tokens, H, top_k)
    L.launch_moe_accum(routed_o, down_o, rows, sw_o, tokens, H)
    out_ro = dev_empty((tokens, H), np.uint16)
    L.launch_moe_round_bf16(out_ro, routed_o, tokens * H)
    sync()

    # the tail, whole and in halves, both accumulation forms
    act, sw, out = dev_empty((tokens, S), np.uint16), dev_empty((tokens,), np.float32), dev_empty((tokens, H), np.uint16)
    L.qwen_moe_shared_tail_decode_fp8(x_d, H, gp, gs, up, us, dp, ds, g_d, act, sw, acc_d, out, tokens, H, S, None, rs, cs)
    sync()
    assert np.array_equal(host(act), host(act_o)) and np.array_equal(host(sw), host(sw_o))
    assert np.array_equal(host(out), host(out_o))
    out.fill_(0x3F01)
    L.qwen_moe_shared_tail_decode_routed_fp8(x_d, H, gp, gs, up, us, dp, ds, g_d, act, sw, contrib_d, weights_d, top_k, out,
                                             tokens, H, S, None, rs, cs)
    sync()
    assert np.array_equal(host(out), host(out_ro))
    act2, sw2, out2 = dev_empty((tokens, S), np.uint16), dev_empty((tokens,), np.float32), dev_empty((tokens, H), np.uint16)
    L.qwen_moe_shared_gate_up_decode_fp8(x_d, H, gp, gs, up, us, g_d, act2, sw2, tokens, H, S, None, rs, cs)
    L.qwen_moe_shared_down_decode_fp8(act2, dp, ds, sw2, acc_d, out2, tokens, H, S, None, rs, cs)
    sync()
    assert np.array_equal(host(act2), host(act_o)) and np.array_equal(host(out2), host(out_o))
    L.qwen_moe_shared_down_decode_routed_fp8(act2, dp, ds, sw2, contrib_d, weights_d, top_k, out2, tokens, H, S, None, rs, cs)
    sync()
    assert np.array_equal(host(out2), host(out_ro))

    # the oracle: strict FP8 dots in double rounded to BF16, SwiGLU without clamps, raw down dots, the gate, one rounding
    (gpp, gss), (upp, uss), (dpp, dss) = mats
    gate64 = orc.gemv_fp8(x, gpp, gss, tokens, S, H, rs, cs)
    up64 = orc.gemv_fp8(x, upp, uss, tokens, S, H, rs, cs)
    gate_b, up_b = orc.bf16_round(gate64), orc.bf16_round(up64)
    act_b = np.empty((tokens, S), dtype=np.uint16)
    orc.oracle().orc_swiglu(orc.p(gate_b), orc.p(up_b), tokens * S, float("inf"), orc.p(act_b))
    down64 = orc.gemv_fp8(act_b, dpp, dss, tokens, H, S, rs, cs)
    ow = np.empty(tokens, dtype=np.float32)
    orc.oracle().orc_shared_gate(orc.p(x), H, orc.p(g), tokens, H, orc.p(ow))
    want = acc.astype(np.float64) + ow.astype(np.float64)[:, None] * down64
    got = np.ascontiguousarray(host(out_o).view(np.uint16))
    want_b = bf16_bits_to_f64(orc.bf16_round(want))
    rep = orc.compare_bf16(got, want_b, 4.0, 2e-2)       # the layer budget: three BF16 rounding points upstream
    assert rep.nan_pattern_errors == 0 and rep.mismatches == 0 and rep.l2_rel < 4e-3, (rep.mismatches, rep.max_ulps, rep.l2_rel)
