"""Small helpers for the GPU parity tests: numpy <-> device buffers through torch (plumbing only)."""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from dgpp_amd import hostgen, launch
from dgpp_amd._lib import Fp4Matrix, MoeExpertView, MoeSegment

DEV = "cuda:0"


def dev(a: np.ndarray) -> torch.Tensor:
    """Uploads a numpy array as raw bytes-compatible torch tensor (uint16 travels as int16)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def dev_empty(shape, dtype) -> torch.Tensor:
    t = {np.uint16: torch.int16, np.float32: torch.float32, np.int32: torch.int32, np.uint8: torch.uint8}[dtype]
    return torch.empty(shape, dtype=t, device=DEV)


def host(t: torch.Tensor, dtype=None) -> np.ndarray:
    a = t.detach().cpu().numpy()
    if dtype is not None and a.dtype != dtype:
        a = a.view(dtype)
    return a


def sync():
    torch.cuda.synchronize()


def fp4_matrix(payload_d, scales_d, global_d, rows, cols, group) -> Fp4Matrix:
    return Fp4Matrix(payload_d.data_ptr(), scales_d.data_ptr(), global_d.data_ptr() if global_d is not None else None,
                     rows, cols, group, 0, None)


def view_table(entries) -> torch.Tensor:
    """Uploads a list of MoeExpertView as the device expert table (96-byte entries)."""
    arr = (MoeExpertView * len(entries))(*entries)
    raw = np.frombuffer(bytes(arr), dtype=np.uint8).copy()
    return torch.from_numpy(raw).to(DEV)


def fp8_view(payload_d, scales_d, rs=7, cs=7) -> MoeExpertView:
    v = MoeExpertView()
    v.payload = payload_d.data_ptr()
    v.scales = scales_d.data_ptr()
    v.scale_shift_rows, v.scale_shift_cols = rs, cs
    v.fp4_group = 16
    return v


def fp4_view(payload_d, scales_d, global_d, group) -> MoeExpertView:
    v = MoeExpertView()
    v.payload = payload_d.data_ptr()
    v.fp4_scales = scales_d.data_ptr()
    v.fp4_global = global_d.data_ptr() if global_d is not None else None
    v.scale_shift_rows, v.scale_shift_cols = 7, 7
    v.fp4_group = group
    return v


def segments_to_numpy(t: torch.Tensor) -> np.ndarray:
    return host(t).view(np.int32).reshape(-1, 3)


class DeviceMoe:
    """A MoeProblem (tests/moe_data.py) uploaded to the GPU: per-matrix tensors and the expert-view table
    ([E * 3] routed entries, then the shared triple when it is an FP4 expert read through the table)."""

    def __init__(self, p):
        self.p = p
        self.keep = []
        entries = []
        for e in p.experts:
            for m in e:
                entries.append(self._view(m))
        self.shared_view_base = -1
        self.sh = None
        if p.shared is not None:
            if p.shared_kind in ("nvfp4", "mxfp4"):
                self.shared_view_base = len(entries)
                for m in p.shared:
                    entries.append(self._view(m))
            else:
                self.sh = [(dev(m.payload), dev(m.scales)) for m in p.shared]
        self.views = view_table(entries)
        self.x = dev(p.x)
        self.fp4_group = 32 if p.kind == "mxfp4" else 16

    def _view(self, m):
        pd, sd = dev(m.payload), dev(m.scales)
        self.keep += [pd, sd]
        if m.kind == "fp8":
            return fp8_view(pd, sd, m.rs, m.cs)
        gd = dev(m.glob) if m.glob is not None else None
        self.keep.append(gd)
        return fp4_view(pd, sd, gd, 16 if m.kind == "nvfp4" else 32)
