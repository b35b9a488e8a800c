"""numpy front-ends of the library's host encoders and seeded generators (C ABI, no GPU).

Weight recipes: block FP8 (src/loaders/fp8_quant.hpp:32-46), NVFP4 (src/loaders/nvfp4_quant.hpp:25-55),
MXFP4 / MXFP8 (ceil-log2 E8M0 byte per 32; src/kernels/latent_format.hpp:117-123).
"""
from __future__ import annotations

import numpy as np

from . import _lib


def _ptr(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def normal_f32(seed: int, shape, std: float = 1.0, mean: float = 0.0, threads: int = 0) -> np.ndarray:
    out = np.empty(shape, dtype=np.float32)
    _lib.load().dgpp_fill_normal_f32(seed, mean, std, out.size, _ptr(out), threads)
    return out


def normal_bf16(seed: int, shape, std: float = 1.0, mean: float = 0.0, threads: int = 0) -> np.ndarray:
    """bf16 bit patterns (uint16) of N(mean, std)."""
    out = np.empty(shape, dtype=np.uint16)
    _lib.load().dgpp_fill_normal_bf16(seed, mean, std, out.size, _ptr(out), threads)
    return out


def f32_to_bf16(a: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even bf16 bit patterns of a float32 array (NaN -> canonical quiet NaN)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) & 0x8000).astype(np.uint16) | 0x7FC0
    return r


def bf16_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def encode_fp8_blocks(w_bf16: np.ndarray, block_rows: int = 128, block_cols: int = 128, threads: int = 0):
    """bf16 bits [rows, cols] -> (payload u8 [rows, cols], scales f32 [ceil(r/br), ceil(c/bc)])."""
    rows, cols = w_bf16.shape
    payload = np.empty((rows, cols), dtype=np.uint8)
    scales = np.empty(((rows + block_rows - 1) // block_rows, (cols + block_cols - 1) // block_cols), dtype=np.float32)
    src = np.ascontiguousarray(w_bf16, dtype=np.uint16)
    _lib.load().dgpp_encode_fp8_blocks(_ptr(src), rows, cols, block_rows, block_cols, _ptr(payload), _ptr(scales), threads)
    return payload, scales


def encode_nvfp4(w: np.ndarray, threads: int = 0):
    """f32 [rows, cols] -> (payload u8 [rows, cols/2], scales e4m3 u8 [rows, cols/16], weight_scale_2).
    The device global the kernels divide by is 1 / weight_scale_2."""
    rows, cols = w.shape
    assert cols % 16 == 0
    payload = np.empty((rows, cols // 2), dtype=np.uint8)
    scales = np.empty((rows, cols // 16), dtype=np.uint8)
    src = np.ascontiguousarray(w, dtype=np.float32)
    ws2 = _lib.load().dgpp_encode_nvfp4(_ptr(src), rows, cols, _ptr(payload), _ptr(scales), threads)
    return payload, scales, float(ws2)


def encode_mxfp4(w: np.ndarray, threads: int = 0):
    """f32 [rows, cols] -> (payload u8 [rows, cols/2], scales e8m0 u8 [rows, cols/32])."""
    rows, cols = w.shape
    assert cols % 32 == 0
    payload = np.empty((rows, cols // 2), dtype=np.uint8)
    scales = np.empty((rows, cols // 32), dtype=np.uint8)
    src = np.ascontiguousarray(w, dtype=np.float32)
    _lib.load().dgpp_encode_mxfp4(_ptr(src), rows, cols, _ptr(payload), _ptr(scales), threads)
    return payload, scales


def encode_mxfp8(w: np.ndarray, threads: int = 0):
    """f32 [rows, cols] -> (payload e4m3 u8 [rows, cols], scales e8m0 u8 [rows, cols/32])."""
    rows, cols = w.shape
    assert cols % 32 == 0
    payload = np.empty((rows, cols), dtype=np.uint8)
    scales = np.empty((rows, cols // 32), dtype=np.uint8)
    src = np.ascontiguousarray(w, dtype=np.float32)
    _lib.load().dgpp_encode_mxfp8(_ptr(src), rows, cols, _ptr(payload), _ptr(scales), threads)
    return payload, scales


def zipf_routes(seed: int, s: float, tokens: int, top_k: int, n_experts: int) -> np.ndarray:
    ids = np.empty((tokens, top_k), dtype=np.int32)
    _lib.load().dgpp_fill_zipf_routes(seed, s, tokens, top_k, n_experts, _ptr(ids))
    return ids
