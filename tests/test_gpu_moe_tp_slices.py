"""The tensor-parallel split of the MoE layer without a second GPU (the reference's
moe_sliced_ranks_fold_matches_unsliced_oracle, tests/cuda/glm_moe_test.cu:683-941, :1762-1816): every rank's slice
of the intermediate dimension - gate / up rows [r * M, (r + 1) * M) and the matching columns of down, cut with the
loader's own slice functions - runs through the layer driver on the one GPU, the ranks' BF16 partial rows are folded
on the host in rank order (fp32 chain from 0, one rounding: the all-reduce's fold) and the result must sit within
the partials' rounding budget of the UNSLICED oracle. A slicing bug (wrong scale block, wrong column origin) is
thousands of times that budget."""
import numpy as np
import pytest

import moe_data
from dgpp_amd import _lib, hostgen as hg, loader as LD
from gpu_util import DeviceMoe, dev, dev_empty, host, sync
from test_gpu_moe_layer import make_layer

pytestmark = pytest.mark.gpu


def rows_slice(m: moe_data.Mat, r0: int, n: int) -> moe_data.Mat:
    """Rows [r0, r0 + n): for block FP8 the start sits on a scale-block boundary (a pointer view in the loader)."""
    if m.kind == "fp8":
        block = 1 << m.rs
        assert r0 % block == 0
        scales = np.ascontiguousarray(m.scales[r0 // block: -(-(r0 + n) // block)])
        return moe_data.Mat("fp8", n, m.cols, np.ascontiguousarray(m.payload[r0:r0 + n]), scales, rs=m.rs, cs=m.cs)
    return moe_data.Mat(m.kind, n, m.cols, np.ascontiguousarray(m.payload[r0:r0 + n]), np.ascontiguousarray(m.scales[r0:r0 + n]),
                        m.glob)


def cols_slice(m: moe_data.Mat, c0: int, n: int) -> moe_data.Mat:
    """Columns [c0, c0 + n) through the loader's copying slices (the FP8 grid re-blocked where the range asks for it)."""
    if m.kind == "fp8":
        whole = LD.QuantMatrix(m.payload.ctypes.data, m.scales.ctypes.data, None, m.rows, m.cols, 1 << m.rs, 1 << m.cs)
        payload, scales, v = LD.quant_slice(whole, 1, c0, n)
        ok, rs, cs = LD.quant_scale_shifts(v)
        assert ok
        return moe_data.Mat("fp8", m.rows, n, payload, scales, rs=rs, cs=cs)
    group = 16 if m.kind == "nvfp4" else 32
    whole = _lib.Fp4Matrix(m.payload.ctypes.data, m.scales.ctypes.data, None, m.rows, m.cols, group, 0, None)
    payload, scales, _ = LD.fp4_cols_slice(whole, c0, n)
    return moe_data.Mat(m.kind, m.rows, n, payload, scales, m.glob)


def bf16_ulp_at(v: np.ndarray) -> np.ndarray:
    """One bf16 ulp at v's magnitude (v = m * 2^e with m in [0.5, 1): the last of 8 bits is 2^(e - 8))."""
    _, e = np.frexp(np.where(v == 0.0, 1e-30, v))
    return np.ldexp(1.0, e - 8)


def fold_ranks(parts):
    acc = np.zeros(parts[0].shape, np.float32)
    for part in parts:
        acc = (acc + hg.bf16_to_f32(part)).astype(np.float32)
    return hg.f32_to_bf16(acc)


CASES = [
    # E, H, I, K, T, kind, world
    (8, 512, 256, 2, 3, "fp8", 2),      # slice 128
    (16, 1024, 512, 4, 2, "fp8", 4),    # slice 128, four ranks
    (8, 512, 512, 2, 4, "fp8", 2),      # slice 256
    (8, 512, 384, 2, 3, "fp8", 2),      # slice 192: the down grid is re-blocked at 64 for rank 1
    (8, 512, 256, 4, 5, "nvfp4", 2),
    (12, 1024, 512, 8, 8, "mxfp4", 4),  # slice 128: four scale groups of 32 per rank
]


@pytest.mark.parametrize("E,H,I,K,T,kind,world", CASES)
def test_sliced_ranks_fold_matches_the_unsliced_oracle(gpu, E, H, I, K, T, kind, world):
    p = moe_data.make_problem(E, H, I, K, T, kind, 0x511 + E + world, shared_kind=None, limit=10.0, std=0.05)
    ids, w, _, _ = moe_data.orc_router(p, 0, 2.5, True)
    _, oracle_bits = moe_data.orc_forward(p, ids, w)
    ids_d, w_d = dev(ids), dev(w)
    M = I // world
    partials = []
    for r in range(world):
        q = moe_data.MoeProblem(E, H, M, K, T, kind, None, M, limit=p.limit)
        q.x, q.router_gate, q.router_bias = p.x, p.router_gate, p.router_bias
        if kind == "fp8" and (r * M) % 128 != 0:
            # a row range that starts inside a scale block is a copying slice too (grid re-blocked)
            def rows(m):
                whole = LD.QuantMatrix(m.payload.ctypes.data, m.scales.ctypes.data, None, m.rows, m.cols, 128, 128)
                payload, scales, v = LD.quant_slice(whole, 0, r * M, M)
                ok, rs, cs = LD.quant_scale_shifts(v)
                assert ok
                return moe_data.Mat("fp8", M, m.cols, payload, scales, rs=rs, cs=cs)
        else:
            def rows(m):
                return rows_slice(m, r * M, M)
        for g, u, dn in p.experts:
            q.experts.append([rows(g), rows(u), cols_slice(dn, r * M, M)])
        # the rank's own oracle: its partial rows before the fold
        _, part_oracle = moe_data.orc_forward(q, ids, w)
        d = DeviceMoe(q)
        layer = make_layer(q, d, 0, 2.5, T)
        out = dev_empty((T, H), np.uint16)
        layer.enqueue_decode_routed(d.x, H, ids_d, w_d, out, T)
        sync()
        slot = host(out, np.uint16).copy()
        out2 = dev_empty((T, H), np.uint16)
        out2.fill_(0x7F7F)
        layer.enqueue_grouped_routed(d.x, H, ids_d, w_d, out2, T)
        sync()
        assert np.array_equal(host(out2, np.uint16), slot), f"rank {r}: the grouped path is bitwise the decode-slot path"
        # each partial is the rank's own oracle to the expert budget's hard bound (12 ulps; measured <= 1)
        po, ps = hg.bf16_to_f32(part_oracle).astype(np.float64), hg.bf16_to_f32(slot).astype(np.float64)
        rms = float(np.sqrt(np.mean(po ** 2)))
        assert np.all(np.abs(ps - po) <= np.maximum(12 * bf16_ulp_at(po), 0.02 * rms)), f"rank {r}: partial rows"
        partials.append(slot)
        layer.close()
    folded = fold_ranks(partials)
    want = hg.bf16_to_f32(oracle_bits).astype(np.float64)
    got = hg.bf16_to_f32(folded).astype(np.float64)
    budget = 0.5 * bf16_ulp_at(want)
    for part in partials:
        budget = budget + 1.5 * bf16_ulp_at(hg.bf16_to_f32(part).astype(np.float64))
    err = np.abs(got - want)
    assert np.all(err <= budget), f"sliced fold: worst err / budget {np.max(err / budget):.3f}"
    l2 = float(np.sqrt(np.sum((got - want) ** 2) / max(np.sum(want ** 2), 1e-300)))
    assert l2 < 4e-3, f"sliced fold: l2 {l2}"
