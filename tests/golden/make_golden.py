"""Writes the small golden fixtures of this folder from the COMPILED REFERENCE oracle
(oracle/_ref/libdgpp_ref.so, built by oracle/Makefile from the reference's own sources).

Run in a container that has the reference checkout:  python tests/golden/make_golden.py
Each .npz holds inputs (quantised weights in the reference's flat layout are re-derivable from the
seeds, so only seeds and shapes are stored) and the reference's outputs: router ids / weights and
the layer's bf16 output. The fixtures let the oracle be checked where the reference is absent.
"""
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent))
sys.path.insert(0, str(HERE.parent.parent))

import moe_data  # noqa: E402
import oracle_lib as orc  # noqa: E402

CASES = [
    # name, E, H, I, K, T, kind, shared_kind, router mode, scaling, norm, limit, seed
    ("fp8_sigmoid", 6, 128, 128, 2, 3, "fp8", "fp8", 0, 2.5, True, 10.0, 11),
    ("nvfp4_sigmoid_fp8shared", 6, 128, 64, 3, 2, "nvfp4", "fp8", 0, 2.5, True, 10.0, 12),
    ("nvfp4_shared_fp4", 5, 64, 64, 2, 3, "nvfp4", "nvfp4", 2, 1.5, True, 7.0, 13),
    ("mxfp4_softmax", 8, 128, 64, 4, 3, "mxfp4", "fp8", 1, 1.0, True, float("inf"), 14),
]


def main():
    assert orc.ref() is not None, "build oracle/_ref first (make -C oracle)"
    for (name, E, H, I, K, T, kind, shared, mode, scaling, norm, limit, seed) in CASES:
        p = moe_data.make_problem(E, H, I, K, T, kind, seed, shared_kind=shared, limit=limit, std=0.05)
        ids, w, biased = moe_data.ref_router(p, mode, scaling, norm)
        out = moe_data.ref_forward(p, mode, scaling, norm)
        np.savez_compressed(HERE / f"moe_{name}.npz", meta=np.array([E, H, I, K, T, mode, seed], np.int64),
                            kind=np.array(kind), shared=np.array(shared), scaling=np.float64(scaling),
                            norm=np.int64(norm), limit=np.float64(limit), x=p.x, router_gate=p.router_gate,
                            router_bias=p.router_bias, ids=ids, weights=w, biased=biased, out=out,
                            digest=np.array([m.payload.sum(dtype=np.uint64) for e in p.experts for m in e], np.uint64))
        print("wrote", name, out.shape)
    # quantiser bytes for seeded inputs (RNE tie cases included)
    r = orc.ref()
    from dgpp_amd import hostgen as hg
    w = hg.normal_f32(77, (9, 96), 0.05)
    w[0, 5] = 0.9
    w[3, :16] = np.array([0, .5, 1, 1.5, 2, 3, 4, 6] * 2, np.float32) * np.float32(0.01)   # on-grid block
    w[4, 16:32] = 0.0
    amax = float(np.abs(w).max())
    ws2 = r.ref_nvfp4_tensor_scale(amax)
    payload = np.empty((9, 48), np.uint8)
    scales = np.empty((9, 6), np.uint8)
    for i in range(9):
        row = np.ascontiguousarray(w[i])
        r.ref_nvfp4_encode_row(orc.p(row), 96, ws2, payload[i].ctypes.data, scales[i].ctypes.data)
    wb = hg.f32_to_bf16(hg.normal_f32(78, (200, 136), 0.02))
    wb[130:, :8] = 0
    p8 = np.empty((200, 136), np.uint8)
    s8 = np.empty((2, 2), np.float32)
    r.ref_fp8_encode_block128(orc.p(wb), 200, 136, orc.p(p8), orc.p(s8))
    np.savez_compressed(HERE / "quantizers.npz", w=w, ws2=np.float32(ws2), nvfp4_payload=payload, nvfp4_scales=scales,
                        wb=wb, fp8_payload=p8, fp8_scales=s8)
    print("wrote quantizers")


if __name__ == "__main__":
    main()
