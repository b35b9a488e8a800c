"""ctypes mirror of include/dgpp_amd_loader.h: the memory-mapped safetensors reader and the quantized
matrix views (reference: src/loaders/safetensors.hpp, src/models/quant_matrix.hpp). Host side only."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib

MAX_RANK = 8
DT_F32, DT_F16, DT_BF16, DT_F8_E4M3, DT_I64, DT_I32, DT_U8, DT_I8, DT_F8_E8M0, DT_U32, DT_I16 = range(11)
_NUMPY = {DT_F32: np.float32, DT_F16: np.float16, DT_BF16: np.uint16, DT_F8_E4M3: np.uint8, DT_I64: np.int64,
          DT_I32: np.int32, DT_U8: np.uint8, DT_I8: np.int8, DT_F8_E8M0: np.uint8, DT_U32: np.uint32, DT_I16: np.int16}


class LoaderError(RuntimeError):
    pass


class TensorInfo(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("rank", C.c_int32), ("shape", C.c_int64 * MAX_RANK), ("numel", C.c_uint64),
                ("nbytes", C.c_uint64), ("file_offset", C.c_uint64), ("data", C.c_void_p)]

    def dims(self):
        return tuple(self.shape[i] for i in range(self.rank))


class QuantMatrix(C.Structure):
    """src/models/quant_matrix.hpp:16-52 (GlmQuantMatrix)."""
    _fields_ = [("payload", C.c_void_p), ("scales", C.c_void_p), ("scales_e8m0", C.c_void_p), ("rows", C.c_int64),
                ("cols", C.c_int64), ("scale_block_rows", C.c_int32), ("scale_block_cols", C.c_int32)]


_P, _I = C.c_void_p, C.c_int
SIGNATURES = {
    "dgpp_loader_last_error": (C.c_char_p, []),
    "dgpp_dtype_size": (C.c_size_t, [_I]),
    "dgpp_safetensors_open": (_I, [C.c_char_p, C.POINTER(_P)]),
    "dgpp_safetensors_close": (None, [_P, _I]),
    "dgpp_safetensors_count": (_I, [_P]),
    "dgpp_safetensors_name": (C.c_char_p, [_P, _I]),
    "dgpp_safetensors_find": (_I, [_P, C.c_char_p, C.POINTER(TensorInfo)]),
    "dgpp_safetensors_header_fold": (C.c_uint64, [_P]),
    "dgpp_safetensors_metadata_json": (C.c_char_p, [_P]),
    "dgpp_safetensors_prefetch": (None, [_P, C.POINTER(TensorInfo)]),
    "dgpp_safetensors_discard": (None, [_P, C.POINTER(TensorInfo)]),
    "dgpp_quant_scale_shifts": (_I, [C.POINTER(QuantMatrix), C.POINTER(_I), C.POINTER(_I)]),
    "dgpp_quant_rows_view": (_I, [C.POINTER(QuantMatrix), C.c_int64, C.c_int64, C.POINTER(QuantMatrix)]),
    "dgpp_fp4_check_cols": (_I, [C.c_int64, _I]),
    "dgpp_fp4_rows_view": (_I, [C.POINTER(_lib.Fp4Matrix), C.c_int64, C.c_int64, C.POINTER(_lib.Fp4Matrix)]),
    "dgpp_quant_slice_scale_count": (C.c_int64, [C.POINTER(QuantMatrix), _I, C.c_int64, C.c_int64]),
    "dgpp_quant_slice": (_I, [C.POINTER(QuantMatrix), _I, C.c_int64, C.c_int64, _P, _P, C.POINTER(QuantMatrix)]),
    "dgpp_fp4_cols_slice": (_I, [C.POINTER(_lib.Fp4Matrix), C.c_int64, C.c_int64, _P, _P, C.POINTER(_lib.Fp4Matrix)]),
    "dgpp_expert_view_from_quant": (_I, [C.POINTER(QuantMatrix), C.POINTER(_lib.MoeExpertView)]),
    "dgpp_expert_view_from_fp4": (_I, [C.POINTER(_lib.Fp4Matrix), C.POINTER(_lib.MoeExpertView)]),
    "dgpp_checkpoint_open": (_I, [C.c_char_p, C.POINTER(_P)]),
    "dgpp_checkpoint_close": (None, [_P]),
    "dgpp_checkpoint_shard_count": (_I, [_P]),
    "dgpp_checkpoint_shards": (C.POINTER(_P), [_P]),
    "dgpp_checkpoint_shard_path": (C.c_char_p, [_P, _I]),
    "dgpp_checkpoint_tensor_count": (C.c_uint64, [_P]),
    "dgpp_checkpoint_find": (_I, [_P, C.c_char_p, C.POINTER(TensorInfo), C.POINTER(_I)]),
}
_typed = False


def lib() -> C.CDLL:
    global _typed
    handle = _lib.load()
    if not _typed:
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _typed = True
    return handle


def _check(rc: int) -> None:
    if rc == _lib.OK:
        return
    msg = lib().dgpp_loader_last_error().decode()
    if rc == _lib.INVALID_ARGUMENT:
        raise ValueError(msg)
    raise LoaderError(msg)


class SafetensorsFile:
    """A mapped checkpoint shard. Arrays returned by `array` alias the mapping: drop them before `close`."""

    def __init__(self, path: str):
        self._h = _P()
        _check(lib().dgpp_safetensors_open(str(path).encode(), C.byref(self._h)))

    def close(self, drop_page_cache: bool = False) -> None:
        if self._h:
            lib().dgpp_safetensors_close(self._h, 1 if drop_page_cache else 0)
            self._h = _P()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __len__(self) -> int:
        return lib().dgpp_safetensors_count(self._h)

    def names(self):
        return [lib().dgpp_safetensors_name(self._h, i).decode() for i in range(len(self))]

    def find(self, name: str) -> TensorInfo:
        info = TensorInfo()
        _check(lib().dgpp_safetensors_find(self._h, name.encode(), C.byref(info)))
        return info

    def __contains__(self, name: str) -> bool:
        info = TensorInfo()
        return lib().dgpp_safetensors_find(self._h, name.encode(), C.byref(info)) == _lib.OK

    def header_fold(self) -> int:
        return lib().dgpp_safetensors_header_fold(self._h)

    def metadata_json(self) -> str:
        return lib().dgpp_safetensors_metadata_json(self._h).decode()

    def prefetch(self, info: TensorInfo) -> None:
        lib().dgpp_safetensors_prefetch(self._h, C.byref(info))

    def discard(self, info: TensorInfo) -> None:
        lib().dgpp_safetensors_discard(self._h, C.byref(info))

    def array(self, name: str) -> np.ndarray:
        """The tensor's bytes as a read-only numpy view of the mapping (bf16 as uint16 bit patterns,
        fp8 / e8m0 as uint8)."""
        info = self.find(name)
        dt = np.dtype(_NUMPY[info.dtype])
        if info.nbytes == 0:
            return np.empty(info.dims(), dtype=dt)
        buf = (C.c_uint8 * info.nbytes).from_address(info.data)
        a = np.frombuffer(buf, dtype=dt).reshape(info.dims())
        a.flags.writeable = False
        return a


class _Shard(SafetensorsFile):
    """A shard a Checkpoint owns: the same accessors, closed with the checkpoint."""

    def __init__(self, handle):
        self._h = handle

    def close(self, drop_page_cache: bool = False) -> None:   # the checkpoint closes it
        self._h = _P()


class Checkpoint:
    """A checkpoint directory as one shard set: the index's weight_map names the shards when there is an index, else
    every *.safetensors file of the directory. `files` is what the bind functions take."""

    def __init__(self, directory: str):
        self._h = _P()
        _check(lib().dgpp_checkpoint_open(str(directory).encode(), C.byref(self._h)))
        n = lib().dgpp_checkpoint_shard_count(self._h)
        arr = lib().dgpp_checkpoint_shards(self._h)
        self.files = [_Shard(_P(arr[i])) for i in range(n)]

    def close(self) -> None:
        if self._h:
            for f in self.files:
                f.close()
            lib().dgpp_checkpoint_close(self._h)
            self._h = _P()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def shard_paths(self):
        return [lib().dgpp_checkpoint_shard_path(self._h, i).decode() for i in range(len(self.files))]

    def tensor_count(self) -> int:
        return int(lib().dgpp_checkpoint_tensor_count(self._h))

    def find(self, name: str):
        """(TensorInfo, shard index); ValueError when no shard has the tensor."""
        info, at = TensorInfo(), _I()
        _check(lib().dgpp_checkpoint_find(self._h, name.encode(), C.byref(info), C.byref(at)))
        return info, at.value

    def array(self, name: str) -> np.ndarray:
        _, at = self.find(name)
        return self.files[at].array(name)


def quant_scale_shifts(m: QuantMatrix):
    rs, cs = _I(), _I()
    ok = lib().dgpp_quant_scale_shifts(C.byref(m), C.byref(rs), C.byref(cs))
    return bool(ok), rs.value, cs.value


def quant_rows_view(m: QuantMatrix, row_start: int, rows: int) -> QuantMatrix:
    out = QuantMatrix()
    _check(lib().dgpp_quant_rows_view(C.byref(m), row_start, rows, C.byref(out)))
    return out


def fp4_rows_view(m, row_start: int, rows: int):
    out = _lib.Fp4Matrix()
    _check(lib().dgpp_fp4_rows_view(C.byref(m), row_start, rows, C.byref(out)))
    return out


def expert_view_from_quant(m: QuantMatrix):
    out = _lib.MoeExpertView()
    _check(lib().dgpp_expert_view_from_quant(C.byref(m), C.byref(out)))
    return out


def expert_view_from_fp4(m):
    out = _lib.MoeExpertView()
    _check(lib().dgpp_expert_view_from_fp4(C.byref(m), C.byref(out)))
    return out


def quant_slice(m: QuantMatrix, axis: int, start: int, count: int):
    """A host copy of a row (axis 0) or column (axis 1) range with the sliced axis' grid re-blocked.
    Returns (payload uint8 [rows, cols], scales float32 [grid], QuantMatrix over them)."""
    n = lib().dgpp_quant_slice_scale_count(C.byref(m), axis, start, count)
    if n < 0:
        n = 0
    rows, cols = (count, m.cols) if axis == 0 else (m.rows, count)
    payload = np.empty((rows, cols) if n else (0, 0), dtype=np.uint8)
    scales = np.empty(n, dtype=np.float32)
    out = QuantMatrix()
    _check(lib().dgpp_quant_slice(C.byref(m), axis, start, count, payload.ctypes.data, scales.ctypes.data, C.byref(out)))
    grid_rows = -(-out.rows // out.scale_block_rows)
    return payload, scales.reshape(grid_rows, -1), out


def fp4_cols_slice(m, col_start: int, cols: int):
    """A host copy of a column range of an NVFP4 / MXFP4 matrix (whole scale groups)."""
    ok = cols > 0 and m.scale_group in (16, 32) and cols % m.scale_group == 0
    payload = np.empty((m.rows, cols // 2) if ok else (0, 0), dtype=np.uint8)
    scales = np.empty((m.rows, cols // m.scale_group) if ok else (0, 0), dtype=np.uint8)
    out = _lib.Fp4Matrix()
    _check(lib().dgpp_fp4_cols_slice(C.byref(m), col_start, cols, payload.ctypes.data, scales.ctypes.data, C.byref(out)))
    return payload, scales, out


BIND_FP8, BIND_NVFP4, BIND_FP8_BF16_SCALES, BIND_NVFP4_MODELOPT, BIND_MXFP8 = 0, 1, 2, 3, 4
BIND_NVFP4_COMPRESSED, BIND_MXFP4, BIND_MXFP8_SCALE_INV = 5, 6, 7


class MoeMatrixTensors(C.Structure):
    """DgppMoeMatrixTensors: where one expert matrix's tensors sit in the shards."""
    _fields_ = [("payload", TensorInfo), ("scales", TensorInfo), ("global_", TensorInfo), ("format", C.c_int32),
                ("file_index", C.c_int32)]


SIGNATURES["dgpp_glm_moe_bind_layer"] = (_I, [C.POINTER(_P), _I, C.c_char_p, _I, C.c_int64, C.c_int64, _I, C.c_int64, _I,
                                               C.POINTER(TensorInfo), C.POINTER(TensorInfo), C.POINTER(MoeMatrixTensors),
                                               C.POINTER(MoeMatrixTensors)])


def glm_moe_bind_layer(files, layer_prefix: str, n_experts: int, hidden: int, inter: int, routed_format: int, shared_inter: int = 0,
                       with_bias: bool = True):
    """The tensors of one GLM-family MoE layer looked up by name across `files` (SafetensorsFile objects) and checked
    against the geometry. Returns (router_weight, router_bias or None, shared [3] or None, routed [n_experts][3])."""
    handles = (_P * len(files))(*[f._h for f in files])
    rw, rb = TensorInfo(), TensorInfo()
    shared = (MoeMatrixTensors * 3)()
    routed = (MoeMatrixTensors * (3 * n_experts))()
    _check(lib().dgpp_glm_moe_bind_layer(handles, len(files), layer_prefix.encode(), n_experts, hidden, inter, routed_format,
                                         shared_inter, 1 if with_bias else 0, C.byref(rw), C.byref(rb) if with_bias else None,
                                         shared if shared_inter > 0 else None, routed))
    return (rw, rb if with_bias else None, list(shared) if shared_inter > 0 else None,
            [[routed[3 * e + m] for m in range(3)] for e in range(n_experts)])


SIGNATURES["dgpp_qwen_moe_bind_layer"] = (_I, [C.POINTER(_P), _I, C.c_char_p, _I, C.c_int64, C.c_int64, _I, C.c_int64, _I,
                                                C.POINTER(TensorInfo), C.POINTER(TensorInfo), C.POINTER(MoeMatrixTensors),
                                                C.POINTER(MoeMatrixTensors)])


def qwen_moe_bind_layer(files, mlp_prefix: str, n_experts: int, hidden: int, inter: int, routed_format: int, shared_inter: int = 0,
                        shared_format: int = BIND_FP8):
    """The tensors of one Qwen-family MoE block. Returns (router_weight, shared_gate or None, shared [3] or None,
    routed [n_experts][3])."""
    handles = (_P * len(files))(*[f._h for f in files])
    rw, sg = TensorInfo(), TensorInfo()
    shared = (MoeMatrixTensors * 3)()
    routed = (MoeMatrixTensors * (3 * n_experts))()
    _check(lib().dgpp_qwen_moe_bind_layer(handles, len(files), mlp_prefix.encode(), n_experts, hidden, inter, routed_format,
                                          shared_inter, shared_format, C.byref(rw), C.byref(sg) if shared_inter > 0 else None,
                                          shared if shared_inter > 0 else None, routed))
    return (rw, sg if shared_inter > 0 else None, list(shared) if shared_inter > 0 else None,
            [[routed[3 * e + m] for m in range(3)] for e in range(n_experts)])


SIGNATURES["dgpp_mimo_moe_bind_layer"] = (_I, [C.POINTER(_P), _I, C.c_char_p, _I, C.c_int64, C.c_int64, C.POINTER(TensorInfo),
                                                C.POINTER(TensorInfo), C.POINTER(MoeMatrixTensors)])
SIGNATURES["dgpp_minimax_moe_bind_layer"] = (_I, [C.POINTER(_P), _I, C.c_char_p, _I, C.c_int64, C.c_int64, C.c_int64,
                                                   C.POINTER(TensorInfo), C.POINTER(TensorInfo), C.POINTER(MoeMatrixTensors),
                                                   C.POINTER(MoeMatrixTensors)])


def mimo_moe_bind_layer(files, mlp_prefix: str, n_experts: int, hidden: int, inter: int):
    """The tensors of one MiMo-family MXFP4 MoE block. Returns (router_weight, router_bias, routed [n_experts][3])."""
    handles = (_P * len(files))(*[f._h for f in files])
    rw, rb = TensorInfo(), TensorInfo()
    routed = (MoeMatrixTensors * (3 * n_experts))()
    _check(lib().dgpp_mimo_moe_bind_layer(handles, len(files), mlp_prefix.encode(), n_experts, hidden, inter, C.byref(rw),
                                          C.byref(rb), routed))
    return rw, rb, [[routed[3 * e + m] for m in range(3)] for e in range(n_experts)]


def minimax_moe_bind_layer(files, moe_prefix: str, n_experts: int, hidden: int, inter: int, shared_inter: int = 0):
    """The tensors of one MiniMax-family MoE block (NVFP4 routed w1 / w3 / w2 as gate / up / down, MXFP8 shared).
    Returns (router_weight, router_bias, shared [3] or None, routed [n_experts][3])."""
    handles = (_P * len(files))(*[f._h for f in files])
    rw, rb = TensorInfo(), TensorInfo()
    shared = (MoeMatrixTensors * 3)()
    routed = (MoeMatrixTensors * (3 * n_experts))()
    _check(lib().dgpp_minimax_moe_bind_layer(handles, len(files), moe_prefix.encode(), n_experts, hidden, inter, shared_inter,
                                             C.byref(rw), C.byref(rb), shared if shared_inter > 0 else None, routed))
    return (rw, rb, list(shared) if shared_inter > 0 else None,
            [[routed[3 * e + m] for m in range(3)] for e in range(n_experts)])

