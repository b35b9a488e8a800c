"""ctypes front-end of the CPU oracle (oracle/liboracle.so) and, where it was built, of the
compiled reference oracle (oracle/_ref/libdgpp_ref.so). Test infrastructure only."""
from __future__ import annotations

import ctypes as C
import sys
import subprocess
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
ORACLE_SO = ROOT / "oracle" / "liboracle.so"
REF_SO = ROOT / "oracle" / "_ref" / "libdgpp_ref.so"

_P, _I, _L, _D, _F = C.c_void_p, C.c_int, C.c_int64, C.c_double, C.c_float


class OrcMatrix(C.Structure):
    _fields_ = [("payload", _P), ("scales_f32", _P), ("scales_u8", _P), ("divisor", _D), ("kind", C.c_int32),
                ("group", C.c_int32), ("rs", C.c_int32), ("cs", C.c_int32)]


class OrcCompare(C.Structure):
    _fields_ = [("l2_rel", _D), ("max_rel", _D), ("max_ulps", _D), ("mismatches", _L), ("nan_pattern_errors", _L),
                ("total", _L)]


_SIG = {
    "orc_bf16_to_f32": (_F, [C.c_uint16]), "orc_f32_to_bf16": (C.c_uint16, [_F]),
    "orc_e4m3_to_f32": (_F, [C.c_uint8]), "orc_f32_to_e4m3": (C.c_uint8, [_F]),
    "orc_e2m1_to_f32": (_F, [C.c_uint8]), "orc_f32_to_e2m1": (C.c_uint8, [_F]),
    "orc_e8m0_to_f32": (_F, [C.c_uint8]), "orc_e8m0_ceil_log2": (C.c_uint8, [_F]),
    "orc_dequant_fp8": (None, [_P, _P, _P, _L, _L, _I, _I, _I, _P]),
    "orc_dequant_fp4": (None, [_P, _P, _I, _L, _L, _P]),
    "orc_gemv_fp8": (None, [_P, _L, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]),
    "orc_gemv_fp4": (None, [_P, _L, _P, _P, _D, _I, _I, _I, _I, _P]),
    "orc_router_scores": (None, [_P, _P, _P, _I, _I, _I, _I, _P, _P]),
    "orc_router_select": (None, [_P, _P, _I, _I, _I, _I, _D, _I, _P, _P]),
    "orc_moe_segment": (None, [_P, _I, _I, _I, _P, _P, _P]),
    "orc_moe_slot_order": (None, [_P, _I, _I, _I, _I, _P, _P]),
    "orc_moe_tile_list": (_I, [_P, _I, _I, _P]),
    "orc_compact_segments": (None, [_P, _P, _I, _I]),
    "orc_swiglu": (None, [_P, _P, _L, _F, _P]),
    "orc_slot_accum": (None, [_P, _P, _I, _I, _I, _I, _P, _P]),
    "orc_accum_ordered": (None, [_P, _L, _P, _P, _P, _I, _I, _I, _I, _P, _P]),
    "orc_moe_forward": (None, [_P, _L, _P, _P, _I, _I, _I, _I, _I, _P, _P, _F, _I, _P, _P]),
    "orc_shared_gate": (None, [_P, _L, _P, _I, _I, _P]),
    "orc_mxfp8_quantize_rows": (None, [_P, _L, _I, _I, _P, _P]),
    "orc_nvfp4_quantize_rows": (None, [_P, _L, _I, _I, C.c_float, _P, _P, _L, _P]),
    "orc_hash_routes": (None, [_P, _P, _P, _I, _I, _I, _I, _F, _I, _P, _P]),
    "orc_minimax_quantize_rows_nvfp4": (None, [_P, _L, _I, _I, _P, _P, _P]),
    "orc_minimax_swiglu_f32": (None, [_P, _P, C.c_int64, _D, _D, _P, _P]),
    "orc_minimax_route_scores": (None, [_P, _P, _I, _I, _I, _F, _P, _P]),
    "orc_minimax_router_scores": (None, [_P, _P, _I, _I, _I, _P]),
    "orc_w4a4_gemm": (None, [_P, _P, _L, _P, _P, _P, C.c_double, _I, _I, _I, _P, _P]),
    "orc_swiglu_oai": (None, [_P, _P, _L, _I, _I, _F, _F, _P, _P]),
    "orc_mxfp8_gemm": (None, [_P, _P, _P, _P, _I, _I, _I, _P, _P]),
    "orc_compare_bf16": (None, [_P, _P, _L, _D, _D, _P]),
    "orc_compare_f32": (None, [_P, _P, _L, _D, _D, _P]),
}

_REF_SIG = {
    "ref_bf16_to_f32": (_F, [C.c_uint16]), "ref_f32_to_bf16": (C.c_uint16, [_F]),
    "ref_e4m3_to_f32": (_F, [C.c_uint8]), "ref_f32_to_e4m3": (C.c_uint8, [_F]),
    "ref_e2m1_to_f32": (_F, [C.c_uint8]), "ref_f32_to_e2m1": (C.c_uint8, [_F]),
    "ref_e8m0_to_f32": (_F, [C.c_uint8]), "ref_e8m0_ceil_log2": (C.c_uint8, [_F]),
    "ref_nvfp4_tensor_scale": (_F, [_F]),
    "ref_nvfp4_encode_row": (None, [_P, _L, _F, _P, _P]),
    "ref_fp8_encode_block128": (None, [_P, _L, _L, _P, _P]),
    "ref_minimax_route": (_I, [_P, _P, _I, _I, _F, _P, _P]),
    "ref_router": (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P, _P, _P]),
    "ref_moe_forward": (_I, [_P, _I, _I, _I, _I, _I, _I, _F, _I, _F, _P, _P, _P, _L, _P, _L, _I, _I, _I, _P, _L, _P,
                             _L, _P, _L, _P]),
    "ref_moe_layer_create": (_P, [_I, _I, _I, _I, _I, _F, _I, _F, _P, _P, _I, _P, _L, _P, _L, _P, _L]),
    "ref_moe_layer_forward": (_I, [_P, _P, _I, _P]),
    "ref_moe_layer_destroy": (None, [_P]),
}

_orc = None
_ref = None


def oracle() -> C.CDLL:
    global _orc
    if _orc is None:
        if not ORACLE_SO.exists():
            subprocess.run(["make", "-C", str(ROOT / "oracle"), "liboracle.so"], check=True, capture_output=True)
        _orc = C.CDLL(str(ORACLE_SO))
        for name, (res, args) in _SIG.items():
            fn = getattr(_orc, name)
            fn.restype, fn.argtypes = res, args
    return _orc


def ref():
    """The compiled reference oracle, or None where it was not built."""
    global _ref
    if _ref is None and REF_SO.exists():
        _ref = C.CDLL(str(REF_SO))
        for name, (res, args) in _REF_SIG.items():
            fn = getattr(_ref, name)
            fn.restype, fn.argtypes = res, args
    return _ref


def p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle inputs must be contiguous"
    # The address outlives this call only if the caller holds the array: a temporary (held by
    # nothing but the call's own stack slot, this frame and getrefcount) would be freed first.
    assert sys.getrefcount(a) > 3, "pass a named array: the address of a temporary dangles before the C call"
    return a.ctypes.data


# ---- numpy-level helpers -----------------------------------------------------------------------------
def gemv_fp8(act, payload, scales, m, n, k, rs=7, cs=7, strict=True, e8m0=False):
    out = np.empty((m, n), dtype=np.float64)
    act = np.ascontiguousarray(act)
    oracle().orc_gemv_fp8(p(act), act.shape[-1] if act.ndim > 1 else k, p(payload), None if e8m0 else p(scales),
                          p(scales) if e8m0 else None, m, n, k, rs, cs, 1 if strict else 0, p(out))
    return out


def gemv_fp4(act, payload, scales, divisor, group, m, n, k):
    out = np.empty((m, n), dtype=np.float64)
    act = np.ascontiguousarray(act)
    oracle().orc_gemv_fp4(p(act), act.shape[-1] if act.ndim > 1 else k, p(payload), p(scales), float(divisor), group,
                          m, n, k, p(out))
    return out


def compare_bf16(got_bits, oracle_f64, ulp_budget=2.0, floor_frac=1e-3) -> OrcCompare:
    rep = OrcCompare()
    got = np.ascontiguousarray(got_bits, dtype=np.uint16).ravel()
    orc = np.ascontiguousarray(oracle_f64, dtype=np.float64).ravel()
    assert got.size == orc.size
    oracle().orc_compare_bf16(p(got), p(orc), got.size, ulp_budget, floor_frac, C.addressof(rep))
    return rep


def compare_f32(got, oracle_f64, ulp_budget=2.0, floor_frac=1e-3) -> OrcCompare:
    rep = OrcCompare()
    g = np.ascontiguousarray(got, dtype=np.float32).ravel()
    orc = np.ascontiguousarray(oracle_f64, dtype=np.float64).ravel()
    assert g.size == orc.size
    oracle().orc_compare_f32(p(g), p(orc), g.size, ulp_budget, floor_frac, C.addressof(rep))
    return rep


def bf16_round(x_f64):
    """fp64 -> bf16 bits the way the oracle rounds (through fp32, RNE)."""
    from dgpp_amd import hostgen
    return hostgen.f32_to_bf16(np.asarray(x_f64, dtype=np.float64).astype(np.float32))


def make_matrix(kind, payload, scales, divisor=1.0, group=16, rs=7, cs=7, e8m0=False) -> OrcMatrix:
    m = OrcMatrix()
    m.payload = p(payload)
    if kind == 0 and not e8m0:
        m.scales_f32 = p(scales)
        m.scales_u8 = None
    else:
        m.scales_f32 = None
        m.scales_u8 = p(scales)
    m.divisor = divisor
    m.kind = kind
    m.group = group
    m.rs, m.cs = rs, cs
    return m


def moe_forward(x, ids, weights, hidden, inter, shared_inter, experts, shared, limit, threads=1):
    """experts: list of OrcMatrix [E*3]; shared: list of 3 or None. Returns (raw f64, bf16 bits)."""
    tokens, top_k = ids.shape
    raw = np.empty((tokens, hidden), dtype=np.float64)
    bits = np.empty((tokens, hidden), dtype=np.uint16)
    ex = (OrcMatrix * len(experts))(*experts)
    sh = (OrcMatrix * 3)(*shared) if shared else None
    x = np.ascontiguousarray(x)
    ids32 = np.ascontiguousarray(ids, dtype=np.int32)
    w32 = np.ascontiguousarray(weights, dtype=np.float32)
    oracle().orc_moe_forward(p(x), x.shape[1], p(ids32), p(w32), tokens, top_k, hidden, inter, shared_inter,
                             C.addressof(ex), C.addressof(sh) if sh else None, limit, threads, p(raw), p(bits))
    return raw, bits


def north_star_rel(got_bits, raw_f64, floor_frac=1e-3) -> float:
    """The north-star measure on BF16 outputs: max over elements of the error BEYOND the output's own
    representational rounding (half a bf16 ulp of the oracle value: up to 2^-8 relative, which no bf16
    result can avoid), relative to max(|oracle|, floor_frac * max|oracle|). Must stay <= 2e-3."""
    from dgpp_amd import hostgen
    o = np.asarray(raw_f64, dtype=np.float64).ravel()
    g = hostgen.bf16_to_f32(np.asarray(got_bits, dtype=np.uint16).ravel()).astype(np.float64)
    ok = np.isfinite(o) & np.isfinite(g)
    if not ok.any():
        return 0.0
    o, g = o[ok], g[ok]
    floor_abs = floor_frac * np.abs(o).max()
    with np.errstate(divide="ignore"):
        expo = np.floor(np.log2(np.abs(o), where=o != 0, out=np.full_like(o, -140.0)))
    half_ulp = np.exp2(expo - 8)
    excess = np.maximum(np.abs(g - o) - half_ulp, 0.0)
    return float((excess / np.maximum(np.abs(o), max(floor_abs, 1e-300))).max())
