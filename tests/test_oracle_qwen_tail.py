"""The shared gate of the oracle against numpy, and the argument rules of the shared expert's decode tail
(src/kernels/qwen_moe.cu:312-326, :377-413, :443-482), which run before anything touches a GPU."""
import ctypes as C

import numpy as np

import mxfp8_data as md
import oracle_lib as orc
from np_ref import bf16_bits_to_f64


def test_shared_gate_oracle():
    rng = np.random.default_rng(3)
    tokens, hidden, stride = 5, 96, 104
    x = md.f32_to_bf16_bits(rng.normal(0, 1, size=(tokens, stride)).astype(np.float32))
    g = md.f32_to_bf16_bits(rng.normal(0, 0.2, size=hidden).astype(np.float32))
    x[0, :hidden] = 0                                   # logit 0 -> 0.5
    x[1, :hidden] = md.f32_to_bf16_bits(np.float32(50.0)) * np.ones(hidden, dtype=np.uint16)
    w = np.empty(tokens, dtype=np.float32)
    orc.oracle().orc_shared_gate(orc.p(x), stride, orc.p(g), tokens, hidden, orc.p(w))
    logit = bf16_bits_to_f64(x[:, :hidden]) @ bf16_bits_to_f64(g)
    logit = bf16_bits_to_f64(md.f32_to_bf16_bits(logit.astype(np.float32)))
    want = bf16_bits_to_f64(md.f32_to_bf16_bits((1 / (1 + np.exp(-logit))).astype(np.float32)))
    assert np.array_equal(w.astype(np.float64), want)
    assert w[0] == 0.5
    one = np.empty(tokens, dtype=np.float32)
    orc.oracle().orc_shared_gate(orc.p(x), stride, None, tokens, hidden, orc.p(one))
    assert np.all(one == 1.0)


def test_tail_launchers_reject_what_the_reference_rejects():
    from dgpp_amd import _lib

    lib = _lib.load()
    buf = (C.c_uint8 * 4096)()
    p = (C.addressof(buf) + 15) & ~15
    ok, bad = 0, 1

    def tail(tokens=1, H=64, S=64, rs=7, cs=7, x=p, stride=None, acc=p):
        return lib.dgpp_qwen_moe_shared_tail_decode_fp8(x, H if stride is None else stride, p, p, p, p, p, p, p, p, p, acc, p,
                                                        tokens, H, S, None, rs, cs)

    def routed(top_k, contrib=p, tokens=1):
        return lib.dgpp_qwen_moe_shared_tail_decode_routed_fp8(p, 64, p, p, p, p, p, p, p, p, p, contrib, p, top_k, p, tokens,
                                                               64, 64, None, 7, 7)

    assert tail(tokens=0) == ok and tail(tokens=-3, H=7) == ok
    assert tail(tokens=9) == bad and b"decode rows" in lib.dgpp_last_error()
    for H, S in ((0, 64), (72, 64), (64, 40), (64, 0)):
        assert tail(H=H, S=S) == bad
    assert tail(cs=3) == bad and b"scale grid" in lib.dgpp_last_error()
    assert tail(rs=-1) == bad and tail(cs=31) == bad
    assert tail(x=p + 8) == bad and tail(stride=60) == bad and tail(stride=68) == bad
    assert tail(acc=None) == bad and b"null pointer" in lib.dgpp_last_error()
    assert routed(0) == bad and routed(17) == bad and routed(8, contrib=None) == bad and b"slots" in lib.dgpp_last_error()
    assert routed(8, tokens=0) == ok
    assert lib.dgpp_qwen_moe_shared_gate_bf16(p, p, p, 0, 12, None) == ok
    assert lib.dgpp_qwen_moe_shared_gate_bf16(p, p, p, 1, 12, None) == bad
    assert lib.dgpp_qwen_moe_shared_gate_bf16(p + 2, p, p, 1, 16, None) == bad
    assert lib.dgpp_qwen_moe_shared_gate_bf16(None, p, p, 1, 16, None) == bad
    assert lib.dgpp_qwen_moe_shared_down_decode_fp8(p, p, p, None, p, p, 1, 64, 64, None, 7, 7) == bad
    assert lib.dgpp_qwen_moe_shared_down_decode_routed_fp8(p, p, p, p, p, p, 20, p, 1, 64, 64, None, 7, 7) == bad
    assert lib.dgpp_qwen_moe_shared_gate_up_decode_fp8(p, 64, p, p, p, p, p, None, p, 1, 64, 64, None, 7, 7) == bad
