"""Seeded synthetic MoE layers for the tests: weights quantised with the library's host encoders
(the published recipes), in numpy; adapters to the oracle, to the compiled reference's flat
layout, and to device expert-view tables."""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

import oracle_lib as orc
from dgpp_amd import hostgen as hg


@dataclass
class Mat:
    kind: str                 # "fp8" | "nvfp4" | "mxfp4" | "mxfp8"
    rows: int
    cols: int
    payload: np.ndarray
    scales: np.ndarray
    glob: np.ndarray | None = None   # NVFP4: f32 [1], the DEVICE global (1 / weight_scale_2)
    rs: int = 7
    cs: int = 7

    def orc(self) -> orc.OrcMatrix:
        if self.kind == "fp8":
            return orc.make_matrix(0, self.payload, self.scales, rs=self.rs, cs=self.cs)
        if self.kind == "mxfp8":
            return orc.make_matrix(0, self.payload, self.scales, rs=0, cs=5, e8m0=True)
        if self.kind == "nvfp4":
            return orc.make_matrix(1, self.payload, self.scales, divisor=float(self.glob[0]), group=16)
        return orc.make_matrix(1, self.payload, self.scales, group=32)


def make_mat(kind: str, rows: int, cols: int, seed: int, std: float = 0.02, block: int = 128) -> Mat:
    w = hg.normal_f32(seed, (rows, cols), std)
    if kind == "fp8":
        payload, scales = hg.encode_fp8_blocks(hg.f32_to_bf16(w), block, block)
        s = int(np.log2(block))
        return Mat(kind, rows, cols, payload, scales, rs=s, cs=s)
    if kind == "mxfp8":
        payload, scales = hg.encode_mxfp8(w)
        return Mat(kind, rows, cols, payload, scales, rs=0, cs=5)
    if kind == "nvfp4":
        payload, scales, ws2 = hg.encode_nvfp4(w)
        return Mat(kind, rows, cols, payload, scales, np.array([1.0 / np.float32(ws2)], dtype=np.float32))
    payload, scales = hg.encode_mxfp4(w)
    return Mat(kind, rows, cols, payload, scales)


@dataclass
class MoeProblem:
    E: int
    H: int
    I: int
    K: int
    T: int
    kind: str
    shared_kind: str | None
    shared_I: int
    experts: list = field(default_factory=list)   # [E][3] Mat: gate, up, down
    shared: list | None = None                     # [3] Mat
    x: np.ndarray | None = None                    # bf16 bits [T, H]
    router_gate: np.ndarray | None = None          # bf16 bits [E, H]
    router_bias: np.ndarray | None = None          # f32 [E]
    limit: float = 10.0

    def orc_experts(self):
        return [m.orc() for e in self.experts for m in e]

    def orc_shared(self):
        return [m.orc() for m in self.shared] if self.shared else None


def make_problem(E, H, I, K, T, kind, seed, shared_kind=None, shared_I=None, limit=10.0, std=0.02) -> MoeProblem:
    shared_I = shared_I if shared_I is not None else I
    p = MoeProblem(E, H, I, K, T, kind, shared_kind, shared_I, limit=limit)
    for e in range(E):
        s = seed * 1000 + e * 3
        p.experts.append([make_mat(kind, I, H, s, std), make_mat(kind, I, H, s + 1, std), make_mat(kind, H, I, s + 2, std)])
    if shared_kind:
        s = seed * 1000 + E * 3
        p.shared = [make_mat(shared_kind, shared_I, H, s, std), make_mat(shared_kind, shared_I, H, s + 1, std),
                    make_mat(shared_kind, H, shared_I, s + 2, std)]
    p.x = hg.normal_bf16(seed * 7 + 1, (T, H))
    p.router_gate = hg.normal_bf16(seed * 7 + 2, (E, H), 1.0 / np.sqrt(H))
    p.router_bias = hg.normal_f32(seed * 7 + 3, (E,), 0.05)
    return p


# ---- the compiled reference's flat layout (src/models/glm/moe_reference.hpp:16-40) ---------------------
def ref_forward(p: MoeProblem, mode: int, scaling: float, norm: bool):
    """Runs the compiled reference's glm_moe_ref_forward; returns bf16 bits [T, H] or None without _ref.
    The reference always runs a shared expert of the routed width."""
    r = orc.ref()
    if r is None:
        return None
    assert p.shared is not None and p.shared_I == p.I
    fp4 = p.kind in ("nvfp4", "mxfp4")
    shared_fp4 = p.shared_kind in ("nvfp4", "mxfp4")
    fp8_mats = ([] if fp4 else [m for e in p.experts for m in e]) + ([] if shared_fp4 else p.shared)
    fp4_mats = ([m for e in p.experts for m in e] if fp4 else []) + (p.shared if shared_fp4 else [])
    payloads = np.concatenate([m.payload.ravel() for m in fp8_mats]) if fp8_mats else np.zeros(0, np.uint8)
    scales = np.concatenate([m.scales.ravel() for m in fp8_mats]) if fp8_mats else np.zeros(0, np.float32)
    fp4_payloads = np.concatenate([m.payload.ravel() for m in fp4_mats]) if fp4_mats else np.zeros(0, np.uint8)
    fp4_scales = np.concatenate([m.scales.ravel() for m in fp4_mats]) if fp4_mats else np.zeros(0, np.uint8)
    group = 32 if p.kind == "mxfp4" else 16
    globs = np.concatenate([m.glob for m in fp4_mats]).astype(np.float32) if (fp4_mats and group == 16) else None
    out = np.empty((p.T, p.H), dtype=np.uint16)
    payloads, scales = np.ascontiguousarray(payloads), np.ascontiguousarray(scales, dtype=np.float32)
    rc = r.ref_moe_forward(orc.p(p.x), p.T, p.H, p.I, p.E, p.K, mode, scaling, 1 if norm else 0, p.limit,
                           orc.p(p.router_gate), orc.p(p.router_bias), orc.p(payloads), payloads.size, orc.p(scales),
                           scales.size, 1 if fp4 else 0, 1 if shared_fp4 else 0, group, orc.p(fp4_payloads),
                           fp4_payloads.size, orc.p(fp4_scales), fp4_scales.size,
                           orc.p(globs) if globs is not None else None, globs.size if globs is not None else 0,
                           orc.p(out))
    assert rc == 0, "the reference oracle threw"
    return out


def ref_router(p: MoeProblem, mode: int, scaling: float, norm: bool):
    r = orc.ref()
    if r is None:
        return None
    ids = np.empty((p.T, p.K), np.int32)
    w = np.empty((p.T, p.K), np.float32)
    biased = np.empty((p.T, p.E), np.float64)
    rc = r.ref_router(orc.p(p.x), orc.p(p.router_gate), orc.p(p.router_bias), mode, p.T, p.E, p.H, p.K, scaling,
                      1 if norm else 0, orc.p(ids), orc.p(w), orc.p(biased))
    assert rc == 0
    return ids, w, biased


def orc_router(p: MoeProblem, mode: int, scaling: float, norm: bool):
    scores = np.empty((p.T, p.E), np.float64)
    biased = np.empty((p.T, p.E), np.float64)
    orc.oracle().orc_router_scores(orc.p(p.x), orc.p(p.router_gate), orc.p(p.router_bias), mode, p.T, p.E, p.H,
                                   orc.p(scores), orc.p(biased))
    ids = np.empty((p.T, p.K), np.int32)
    w = np.empty((p.T, p.K), np.float32)
    orc.oracle().orc_router_select(orc.p(scores), orc.p(biased), mode, p.T, p.E, p.K, scaling, 1 if norm else 0,
                                   orc.p(ids), orc.p(w))
    return ids, w, scores, biased


def orc_forward(p: MoeProblem, ids, weights, threads=1):
    return orc.moe_forward(p.x, ids, weights, p.H, p.I, p.shared_I, p.orc_experts(), p.orc_shared(), p.limit, threads)
