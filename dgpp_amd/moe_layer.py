"""Python handle on the C++ host layer driver (dgpp_amd/csrc/moe_layer.cpp, include/dgpp_amd_layer.h),
the counterpart of the reference's GlmMoeLayer (src/models/glm/moe_layer.hpp:50). Tests and the
benchmark drive the decode path through it; pointers are torch tensors / ints as in dgpp_amd.launch."""
from __future__ import annotations

import ctypes as C

from . import _lib
from ._lib import MoeConfig, MoeExpertView, MoeLayerDesc, MoeResidentDesc
from .launch import InvalidArgument, _p, _stream

EXPERTS_FP8, EXPERTS_NVFP4, EXPERTS_MXFP4 = 0, 1, 2


def _check(rc: int) -> None:
    if rc == _lib.OK:
        return
    msg = _lib.load().dgpp_moe_layer_last_error().decode()
    if rc == _lib.INVALID_ARGUMENT:
        raise InvalidArgument(msg)
    raise RuntimeError(msg)


def scratch_bytes(cfg: MoeConfig, max_tokens: int, shared_inter: int = 0, dense_shared: bool = False) -> int:
    if dense_shared:
        return _lib.load().dgpp_moe_layer_scratch_bytes_dense_shared(C.addressof(cfg), max_tokens, shared_inter)
    return _lib.load().dgpp_moe_layer_scratch_bytes(C.addressof(cfg), max_tokens, shared_inter)


class MoeLayer:
    """Owns the layer's device scratch and expert table; every enqueue_* is asynchronous on `stream`."""

    def __init__(self, cfg: MoeConfig, expert_format: int, views: list[MoeExpertView], max_tokens: int, *,
                 shared_in_table: bool = False, shared_inter: int = 0, sh_payload=(None, None, None),
                 sh_scales=(None, None, None), sh_rs: int = 7, sh_cs: int = 7, router_gate=None, router_bias=None,
                 sh_scales_e8m0=(None, None, None)):
        self._lib = _lib.load()
        arr = (MoeExpertView * len(views))(*views)
        d = MoeLayerDesc()
        d.cfg = cfg
        d.expert_format = expert_format
        d.max_tokens = max_tokens
        d.views = C.addressof(arr)
        d.shared_in_table = 1 if shared_in_table else 0
        d.shared_inter = shared_inter
        for i in range(3):
            d.sh_payload[i] = _p(sh_payload[i])
            d.sh_scales[i] = _p(sh_scales[i])
            d.sh_scales_e8m0[i] = _p(sh_scales_e8m0[i])    # all three given: an MXFP8 shared expert run as dense projections
        d.sh_rs, d.sh_cs = sh_rs, sh_cs
        d.router_gate = _p(router_gate)
        d.router_bias = _p(router_bias)
        self.cfg = cfg
        self._keep = (sh_payload, sh_scales, router_gate, router_bias, sh_scales_e8m0)
        handle = C.c_void_p()
        _check(self._lib.dgpp_moe_layer_create(C.addressof(d), C.addressof(handle)))
        self._h = handle

    def close(self):
        if getattr(self, "_h", None):
            self._lib.dgpp_moe_layer_destroy(self._h)
            self._h = None

    __del__ = close

    def enqueue_decode(self, x, x_stride, out_bf16, tokens, stream=None, out_f32=None):
        _check(self._lib.dgpp_moe_layer_enqueue_decode(self._h, _p(x), x_stride, _p(out_bf16), _p(out_f32), tokens,
                                                       _stream(stream)))

    def enqueue_decode_scores(self, x, x_stride, scores, biased, out_bf16, tokens, stream=None, out_f32=None):
        _check(self._lib.dgpp_moe_layer_enqueue_decode_scores(self._h, _p(x), x_stride, _p(scores), _p(biased),
                                                              _p(out_bf16), _p(out_f32), tokens, _stream(stream)))

    def enqueue_decode_routed(self, x, x_stride, ids, weights, out_bf16, tokens, stream=None, out_f32=None):
        _check(self._lib.dgpp_moe_layer_enqueue_decode_routed(self._h, _p(x), x_stride, _p(ids), _p(weights),
                                                              _p(out_bf16), _p(out_f32), tokens, _stream(stream)))

    def check(self, stream=None):
        """Synchronizes the stream; raises when a one-launch expert chain on it gave up its bounded wait."""
        _check(self._lib.dgpp_moe_layer_check(self._h, _stream(stream)))

    def enqueue_grouped_routed(self, x, x_stride, ids, weights, out_bf16, tokens, stream=None, out_f32=None):
        _check(self._lib.dgpp_moe_layer_enqueue_grouped_routed(self._h, _p(x), x_stride, _p(ids), _p(weights),
                                                               _p(out_bf16), _p(out_f32), tokens, _stream(stream)))

    def enqueue_prefill_routed(self, x, x_stride, ids, weights, out_bf16, tokens, stream=None, out_f32=None):
        _check(self._lib.dgpp_moe_layer_enqueue_prefill_routed(self._h, _p(x), x_stride, _p(ids), _p(weights),
                                                               _p(out_bf16), _p(out_f32), tokens, _stream(stream)))

    def enqueue_prefill(self, x, x_stride, out_bf16, tokens, stream=None, out_f32=None):
        _check(self._lib.dgpp_moe_layer_enqueue_prefill(self._h, _p(x), x_stride, _p(out_bf16), _p(out_f32), tokens,
                                                        _stream(stream)))

    def route_prefill_rows(self, x, x_stride, r0, rows, stream=None):
        _check(self._lib.dgpp_moe_layer_route_prefill_rows(self._h, _p(x), x_stride, r0, rows, _stream(stream)))

    def enqueue_prefill_phased(self, x, x_stride, tokens, stream=None):
        _check(self._lib.dgpp_moe_layer_enqueue_prefill_phased(self._h, _p(x), x_stride, tokens, _stream(stream)))

    def accumulate_prefill_rows(self, out_bf16, tokens, r0, rows, stream=None, out_f32=None):
        _check(self._lib.dgpp_moe_layer_accumulate_prefill_rows(self._h, _p(out_bf16), _p(out_f32), tokens, r0, rows,
                                                                _stream(stream)))

    def enqueue_prefill_routed_w4a4(self, x, x_stride, ids, weights, out_bf16, tokens, stream=None, out_f32=None,
                                    act_scales_dev=None, f32_down=False):
        _check(self._lib.dgpp_moe_layer_enqueue_prefill_routed_w4a4(self._h, _p(x), x_stride, _p(ids), _p(weights),
                                                                    _p(out_bf16), _p(out_f32), tokens, _stream(stream),
                                                                    _p(act_scales_dev), int(bool(f32_down))))

    @property
    def views_ptr(self) -> int:
        """Device address of the layer's expert table."""
        return self._lib.dgpp_moe_layer_views(self._h)

    @property
    def ids_ptr(self) -> int:
        return self._lib.dgpp_moe_layer_ids(self._h)

    @property
    def weights_ptr(self) -> int:
        return self._lib.dgpp_moe_layer_weights(self._h)


class ResidentMoeLayer(MoeLayer):
    """A layer made resident from what a loader.*_moe_bind_layer call found: this rank's slices of the expert matrices
    (gate / up rows [rank * inter / world, ...), the matching columns of down) are uploaded into one device allocation
    that the object owns together with the layer driver over it. The shards must be open during construction only."""

    def __init__(self, cfg: MoeConfig, max_tokens: int, routed, *, shared=None, shared_inter: int = 0, router_weight=None,
                 router_bias=None, rank: int = 0, world: int = 1):
        from .loader import MoeMatrixTensors
        self._lib = _lib.load()
        flat = [m for expert in routed for m in expert]
        r_arr = (MoeMatrixTensors * len(flat))(*flat)
        s_arr = (MoeMatrixTensors * 3)(*shared) if shared else None
        d = MoeResidentDesc()
        d.cfg = cfg
        d.max_tokens, d.rank, d.world = max_tokens, rank, world
        d.routed = C.addressof(r_arr)
        d.shared = C.addressof(s_arr) if s_arr is not None else None
        d.shared_inter = shared_inter if shared else 0
        d.router_weight = C.addressof(router_weight) if router_weight is not None else None
        d.router_bias = C.addressof(router_bias) if router_bias is not None else None
        handle = C.c_void_p()
        rc = self._lib.dgpp_moe_resident_load(C.addressof(d), C.addressof(handle))
        if rc != 0:
            msg = self._lib.dgpp_moe_resident_last_error().decode()
            raise InvalidArgument(msg) if rc == 1 else RuntimeError(msg)
        self._resident = handle
        self._h = C.c_void_p(self._lib.dgpp_moe_resident_layer(handle))
        self.cfg = cfg
        self.weight_bytes = self._lib.dgpp_moe_resident_weight_bytes(handle)
        self.inter = self._lib.dgpp_moe_resident_inter(handle)

    def close(self):
        if getattr(self, "_resident", None):
            self._lib.dgpp_moe_resident_destroy(self._resident)   # the layer goes with it
            self._resident = None
            self._h = None

    __del__ = close
