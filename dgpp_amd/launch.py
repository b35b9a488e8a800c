"""Python mirror of the reference's `dgpp::launch_*` operator surface over the C ABI.

Same names, argument order and meaning as the reference headers (src/kernels/glm_moe_launch.hpp,
fp4_gemv.hpp, scale_gemm.hpp, fp8_dequant.hpp, minimax.hpp); the reference's
std::invalid_argument becomes InvalidArgument (a ValueError), its std::runtime_error a
RuntimeError. Pointer arguments accept torch tensors (their data_ptr()), ints or None; torch
only supplies device memory and streams here.
"""
from __future__ import annotations

import ctypes as C

from . import _lib
from ._lib import Fp4Matrix, Fp8GemvProblem, MoeConfig, MoeExpertView, MoeSegment, MoeTile  # noqa: F401

ROUTER_SIGMOID_BIAS, ROUTER_SOFTMAX_TOPK, ROUTER_SQRT_SOFTPLUS_BIAS = 0, 1, 2
K_FP4_GROUP, K_MXFP4_GROUP = 16, 32


class InvalidArgument(ValueError):
    """The reference launcher would have thrown std::invalid_argument; nothing was launched."""


def _p(x):
    if x is None:
        return None
    if isinstance(x, int):
        return x
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    if isinstance(x, (C.Structure, C.Array)):
        return C.addressof(x)
    raise TypeError(f"cannot take a pointer of {type(x)!r}")


def _stream(stream):
    if stream is None:
        return None
    if isinstance(stream, int):
        return stream or None
    return stream.cuda_stream or None  # torch.cuda.Stream


def _check(rc: int) -> None:
    if rc == _lib.OK:
        return
    msg = _lib.load().dgpp_last_error().decode()
    if rc == _lib.INVALID_ARGUMENT:
        raise InvalidArgument(msg)
    raise RuntimeError(msg)


def make_config(hidden, inter, n_experts, top_k, *, n_shared_experts=1, routed_scaling_factor=2.5,
                norm_topk_prob=True, swiglu_limit=10.0, router_mode=ROUTER_SIGMOID_BIAS) -> MoeConfig:
    return MoeConfig(hidden, inter, n_experts, top_k, n_shared_experts, routed_scaling_factor,
                     1 if norm_topk_prob else 0, swiglu_limit, router_mode)


def validate_config(cfg: MoeConfig) -> None:
    _check(_lib.load().dgpp_moe_config_validate(C.addressof(cfg)))


# ---- router -------------------------------------------------------------------------------------
def launch_moe_router(hidden, gate, bias, ids, weights, scores, biased, cfg: MoeConfig, tokens, stream=None,
                      counters=None, allow_tiled=True):
    _check(_lib.load().dgpp_launch_moe_router(_p(hidden), _p(gate), _p(bias), _p(ids), _p(weights), _p(scores),
                                              _p(biased), C.addressof(cfg), tokens, _stream(stream), _p(counters),
                                              1 if allow_tiled else 0))


def dense_fp4_decode_shape(m, n, k, fp4_group=16) -> bool:
    return bool(_lib.load().dgpp_dense_fp4_decode_shape(m, n, k, fp4_group))


def try_dense_fp4_decode_bf16(act, act_stride, seg, views, which, out, m, n, k, stream=None, fp4_group=16) -> bool:
    launched = C.c_int(0)
    _check(_lib.load().dgpp_try_dense_fp4_decode_bf16(_p(act), act_stride, _p(seg), _p(views), which, _p(out), m, n, k,
                                                      _stream(stream), fp4_group, C.addressof(launched)))
    return bool(launched.value)


def launch_scale_gemm_tile_bf16(act, act_stride, w, scales, out, m, n, k, stream=None, rs=7, cs=7):
    _check(_lib.load().dgpp_launch_scale_gemm_tile_bf16(_p(act), act_stride, _p(w), _p(scales), _p(out), m, n, k, _stream(stream), rs, cs))


def launch_scale_gemm_tile_f32(act, act_stride, w, scales, out, m, n, k, stream=None, rs=7, cs=7):
    _check(_lib.load().dgpp_launch_scale_gemm_tile_f32(_p(act), act_stride, _p(w), _p(scales), _p(out), m, n, k, _stream(stream), rs, cs))


def launch_moe_hash_routes(tokens, tid2eid, scores, ids, weights, cfg: MoeConfig, vocab, n_tokens, stream=None):
    _check(_lib.load().dgpp_launch_moe_hash_routes(_p(tokens), _p(tid2eid), _p(scores), _p(ids), _p(weights), C.addressof(cfg),
                                                   vocab, n_tokens, _stream(stream)))


def launch_moe_router_dots(hidden, gate, bias, scores, biased, cfg: MoeConfig, tokens, stream=None):
    """Extension: the router's score rows without the selection."""
    _check(_lib.load().dgpp_launch_moe_router_dots(_p(hidden), _p(gate), _p(bias), _p(scores), _p(biased), C.addressof(cfg),
                                                   tokens, _stream(stream)))


def launch_moe_router_select(scores, biased, ids, weights, cfg: MoeConfig, tokens, stream=None):
    _check(_lib.load().dgpp_launch_moe_router_select(_p(scores), _p(biased), _p(ids), _p(weights), C.addressof(cfg),
                                                     tokens, _stream(stream)))


def launch_moe_router_select_order(scores, biased, ids, weights, order, cfg: MoeConfig, tokens, shared_early=False,
                                   stream=None):
    """Extension: selection + slot order in one launch (order may be None)."""
    _check(_lib.load().dgpp_launch_moe_router_select_order(_p(scores), _p(biased), _p(ids), _p(weights), _p(order),
                                                           C.addressof(cfg), tokens, 1 if shared_early else 0,
                                                           _stream(stream)))


def launch_moe_select_gate_up_swiglu(scores, biased, ids, weights, cfg: MoeConfig, tokens, x, x_stride, views, n_routed,
                                     k_routed, act, act_stride, limit, stream=None):
    """Extension: selection + routed FP8 gate/up in one launch (ids and weights are outputs)."""
    _check(_lib.load().dgpp_launch_moe_select_gate_up_swiglu(_p(scores), _p(biased), _p(ids), _p(weights), C.addressof(cfg),
                                                             tokens, _p(x), x_stride, _p(views), n_routed, k_routed, _p(act),
                                                             act_stride, limit, _stream(stream)))


def launch_moe_select_gate_up_swiglu_fp4(scores, biased, ids, weights, cfg: MoeConfig, tokens, x, x_stride, views, n_routed,
                                         k_routed, act, act_stride, limit, stream=None, fp4_group=16):
    """Extension: selection + routed NVFP4 / MXFP4 gate/up in one launch (ids and weights are outputs)."""
    _check(_lib.load().dgpp_launch_moe_select_gate_up_swiglu_fp4(_p(scores), _p(biased), _p(ids), _p(weights),
                                                                 C.addressof(cfg), tokens, _p(x), x_stride, _p(views),
                                                                 n_routed, k_routed, _p(act), act_stride, limit,
                                                                 _stream(stream), fp4_group))


# ---- elementwise --------------------------------------------------------------------------------
def launch_moe_swiglu_clamp(gate, up, out, n, limit, stream=None):
    _check(_lib.load().dgpp_launch_moe_swiglu_clamp(_p(gate), _p(up), _p(out), n, limit, _stream(stream)))


def launch_moe_gather_rows(src, rows, dst, n_rows, hidden, stream=None):
    _check(_lib.load().dgpp_launch_moe_gather_rows(_p(src), _p(rows), _p(dst), n_rows, hidden, _stream(stream)))


def launch_moe_accum(acc, y, rows, row_weights, n_rows, hidden, stream=None):
    _check(_lib.load().dgpp_launch_moe_accum(_p(acc), _p(y), _p(rows), _p(row_weights), n_rows, hidden, _stream(stream)))


def launch_moe_round_bf16(out, acc, n, stream=None):
    _check(_lib.load().dgpp_launch_moe_round_bf16(_p(out), _p(acc), n, _stream(stream)))


# ---- grouping -------------------------------------------------------------------------------------
def launch_moe_segment(ids, tokens, top_k, n_experts, rows, slot_row, segs, stream=None):
    _check(_lib.load().dgpp_launch_moe_segment(_p(ids), tokens, top_k, n_experts, _p(rows), _p(slot_row), _p(segs),
                                               _stream(stream)))


def moe_tile_list_capacity(n_segs, total_rows, tile_rows) -> int:
    return _lib.load().dgpp_moe_tile_list_capacity(n_segs, total_rows, tile_rows)


def launch_moe_tile_list(segs, n_segs, tile_rows, tiles, count, stream=None):
    _check(_lib.load().dgpp_launch_moe_tile_list(_p(segs), n_segs, tile_rows, _p(tiles), _p(count), _stream(stream)))


def moe_run_groups_max(slots) -> int:
    return _lib.load().dgpp_moe_run_groups_max(slots)


def launch_moe_slot_order(ids, order, slots, top_k, n_experts, stream=None, shared_early=False, runs=None):
    _check(_lib.load().dgpp_launch_moe_slot_order(_p(ids), _p(order), slots, top_k, n_experts, _stream(stream),
                                                  1 if shared_early else 0, _p(runs)))


def minimax_router(x, gate, bias, rows, hidden, experts, topk, factor, scores, ids, weights, stream=None):
    """src/kernels/minimax.hpp:56-60: FP32 gate, sigmoid scores, bias for the ranking only, FP32 weights."""
    _check(_lib.load().dgpp_minimax_router(_p(x), _p(gate), _p(bias), rows, hidden, experts, topk, factor, _p(scores), _p(ids),
                                           _p(weights), _stream(stream)))


def minimax_compact_segments(input, output, experts, capacity, stream=None):
    _check(_lib.load().dgpp_minimax_compact_segments(_p(input), _p(output), experts, capacity, _stream(stream)))


# ---- accumulation -----------------------------------------------------------------------------------
def launch_moe_accum_ordered(out, down, down_stride, slot_row, slot_ids, slot_w, shared_row0, tokens, top_k, hidden,
                             stream=None):
    _check(_lib.load().dgpp_launch_moe_accum_ordered(_p(out), _p(down), down_stride, _p(slot_row), _p(slot_ids),
                                                     _p(slot_w), shared_row0, tokens, top_k, hidden, _stream(stream)))


def launch_moe_accum_ordered_f32(out, down, down_stride, slot_row, slot_ids, slot_w, shared_row0, tokens, top_k,
                                 hidden, stream=None):
    _check(_lib.load().dgpp_launch_moe_accum_ordered_f32(_p(out), _p(down), down_stride, _p(slot_row), _p(slot_ids),
                                                         _p(slot_w), shared_row0, tokens, top_k, hidden,
                                                         _stream(stream)))


def launch_moe_slot_accum(out, contrib, weights, tokens, hidden, top_k, stream=None):
    _check(_lib.load().dgpp_launch_moe_slot_accum(_p(out), _p(contrib), _p(weights), tokens, hidden, top_k,
                                                  _stream(stream)))


def launch_moe_slot_accum_routed_f32(out, contrib, weights, tokens, hidden, top_k, stream=None):
    _check(_lib.load().dgpp_launch_moe_slot_accum_routed_f32(_p(out), _p(contrib), _p(weights), tokens, hidden, top_k,
                                                             _stream(stream)))


def launch_moe_slot_accum_routed_bf16(out, contrib, weights, tokens, hidden, top_k, stream=None):
    """launch_moe_slot_accum_routed_f32 + launch_moe_round_bf16 in one launch (no reference counterpart)."""
    _check(_lib.load().dgpp_launch_moe_slot_accum_routed_bf16(_p(out), _p(contrib), _p(weights), tokens, hidden, top_k,
                                                              _stream(stream)))


# ---- decode-slot kernels ------------------------------------------------------------------------------
def launch_moe_slot_gate_up_swiglu(x, x_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                   sh_gate_payload, sh_gate_scales, sh_up_payload, sh_up_scales, act, act_stride,
                                   slots, top_k, limit, stream=None, sh_rs=7, sh_cs=7):
    _check(_lib.load().dgpp_launch_moe_slot_gate_up_swiglu(
        _p(x), x_stride, _p(ids), _p(order), _p(views), n_routed, k_routed, n_shared, k_shared, _p(sh_gate_payload),
        _p(sh_gate_scales), _p(sh_up_payload), _p(sh_up_scales), _p(act), act_stride, slots, top_k, limit,
        _stream(stream), sh_rs, sh_cs))


def launch_moe_slot_down(act, act_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared, sh_payload,
                         sh_scales, out, out_stride, slots, top_k, stream=None, sh_rs=7, sh_cs=7):
    _check(_lib.load().dgpp_launch_moe_slot_down(
        _p(act), act_stride, _p(ids), _p(order), _p(views), n_routed, k_routed, n_shared, k_shared, _p(sh_payload),
        _p(sh_scales), _p(out), out_stride, slots, top_k, _stream(stream), sh_rs, sh_cs))


def launch_moe_slot_gate_up_swiglu_fp4(x, x_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                       sh_gate_payload, sh_gate_scales, sh_up_payload, sh_up_scales, act, act_stride,
                                       slots, top_k, limit, stream=None, shared_view_base=-1, fp4_group=16, sh_rs=7,
                                       sh_cs=7):
    _check(_lib.load().dgpp_launch_moe_slot_gate_up_swiglu_fp4(
        _p(x), x_stride, _p(ids), _p(order), _p(views), n_routed, k_routed, n_shared, k_shared, _p(sh_gate_payload),
        _p(sh_gate_scales), _p(sh_up_payload), _p(sh_up_scales), _p(act), act_stride, slots, top_k, limit,
        _stream(stream), shared_view_base, fp4_group, sh_rs, sh_cs))


def launch_moe_slot_down_fp4(act, act_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared, sh_payload,
                             sh_scales, out, out_stride, slots, top_k, stream=None, shared_view_base=-1, fp4_group=16,
                             sh_rs=7, sh_cs=7, tile_counter=None):
    _check(_lib.load().dgpp_launch_moe_slot_down_fp4(
        _p(act), act_stride, _p(ids), _p(order), _p(views), n_routed, k_routed, n_shared, k_shared, _p(sh_payload),
        _p(sh_scales), _p(out), out_stride, slots, top_k, _stream(stream), shared_view_base, fp4_group, sh_rs, sh_cs,
        _p(tile_counter)))


def launch_moe_slot_gate_up_swiglu_mixed(x, x_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared, sh_gate_payload,
                                         sh_gate_scales, sh_up_payload, sh_up_scales, act, act_stride, slots, top_k, limit,
                                         gate_fp4, fp4_group=16, stream=None, sh_rs=7, sh_cs=7):
    _check(_lib.load().dgpp_launch_moe_slot_gate_up_swiglu_mixed(
        _p(x), x_stride, _p(ids), _p(order), _p(views), n_routed, k_routed, n_shared, k_shared, _p(sh_gate_payload),
        _p(sh_gate_scales), _p(sh_up_payload), _p(sh_up_scales), _p(act), act_stride, slots, top_k, limit,
        1 if gate_fp4 else 0, fp4_group, _stream(stream), sh_rs, sh_cs))


def launch_moe_slot_gate_up_swiglu_ex(x, x_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                      sh_gate_payload, sh_gate_scales, sh_up_payload, sh_up_scales, act, act_stride,
                                      slots, top_k, limit, stream=None, sh_rs=7, sh_cs=7, passes=3):
    """Extension: the launcher above with the pass selector as an argument (1 routed, 2 shared, 3 both)."""
    _check(_lib.load().dgpp_launch_moe_slot_gate_up_swiglu_ex(
        _p(x), x_stride, _p(ids), _p(order), _p(views), n_routed, k_routed, n_shared, k_shared, _p(sh_gate_payload),
        _p(sh_gate_scales), _p(sh_up_payload), _p(sh_up_scales), _p(act), act_stride, slots, top_k, limit,
        _stream(stream), sh_rs, sh_cs, passes))


def launch_moe_slot_down_ex(act, act_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared, sh_payload,
                            sh_scales, out, out_stride, slots, top_k, stream=None, sh_rs=7, sh_cs=7, passes=3,
                            acc_weights=None, acc_out=None):
    """Extension: pass selector, and the accumulation the shared pass ends with (both or neither of acc_*)."""
    _check(_lib.load().dgpp_launch_moe_slot_down_ex(
        _p(act), act_stride, _p(ids), _p(order), _p(views), n_routed, k_routed, n_shared, k_shared, _p(sh_payload),
        _p(sh_scales), _p(out), out_stride, slots, top_k, _stream(stream), sh_rs, sh_cs, passes, _p(acc_weights),
        _p(acc_out)))


def launch_moe_slot_gate_up_swiglu_fp4_ex(x, x_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared,
                                          sh_gate_payload, sh_gate_scales, sh_up_payload, sh_up_scales, act, act_stride,
                                          slots, top_k, limit, stream=None, shared_view_base=-1, fp4_group=16, sh_rs=7,
                                          sh_cs=7, passes=3):
    _check(_lib.load().dgpp_launch_moe_slot_gate_up_swiglu_fp4_ex(
        _p(x), x_stride, _p(ids), _p(order), _p(views), n_routed, k_routed, n_shared, k_shared, _p(sh_gate_payload),
        _p(sh_gate_scales), _p(sh_up_payload), _p(sh_up_scales), _p(act), act_stride, slots, top_k, limit,
        _stream(stream), shared_view_base, fp4_group, sh_rs, sh_cs, passes))


def launch_moe_slot_down_fp4_ex(act, act_stride, ids, order, views, n_routed, k_routed, n_shared, k_shared, sh_payload,
                                sh_scales, out, out_stride, slots, top_k, stream=None, shared_view_base=-1, fp4_group=16,
                                sh_rs=7, sh_cs=7, tile_counter=None, passes=3, acc_weights=None, acc_out=None):
    _check(_lib.load().dgpp_launch_moe_slot_down_fp4_ex(
        _p(act), act_stride, _p(ids), _p(order), _p(views), n_routed, k_routed, n_shared, k_shared, _p(sh_payload),
        _p(sh_scales), _p(out), out_stride, slots, top_k, _stream(stream), shared_view_base, fp4_group, sh_rs, sh_cs,
        _p(tile_counter), passes, _p(acc_weights), _p(acc_out)))


def launch_moe_slot_down_accum(act, act_stride, ids, views, n, k, tokens, top_k, weights, out_bf16, out_f32, stream=None):
    """Extension: routed down rows + the ordered accumulation in one token-major launch (FP8 experts)."""
    _check(_lib.load().dgpp_launch_moe_slot_down_accum(_p(act), act_stride, _p(ids), _p(views), n, k, tokens, top_k,
                                                       _p(weights), _p(out_bf16), _p(out_f32), _stream(stream)))


def launch_moe_slot_down_accum_fp4(act, act_stride, ids, views, n, k, tokens, top_k, weights, out_bf16, out_f32,
                                   stream=None, fp4_group=16):
    """Extension: routed down rows + the ordered accumulation in one token-major launch (NVFP4 / MXFP4 experts)."""
    _check(_lib.load().dgpp_launch_moe_slot_down_accum_fp4(_p(act), act_stride, _p(ids), _p(views), n, k, tokens, top_k,
                                                           _p(weights), _p(out_bf16), _p(out_f32), _stream(stream),
                                                           fp4_group))


def moe_slot_chain_ready_bytes(tokens, top_k):
    return int(_lib.load().dgpp_moe_slot_chain_ready_bytes(tokens, top_k))


def launch_moe_slot_chain(x, x_stride, ids, views, inter, hidden, act, act_stride, tokens, top_k, limit, weights, out_bf16,
                          out_f32, ready, status, spins=0, stream=None):
    """Extension: the routed chain (gate/up + SwiGLU, down, accumulation) of a small decode batch in one launch (FP8)."""
    _check(_lib.load().dgpp_launch_moe_slot_chain(_p(x), x_stride, _p(ids), _p(views), inter, hidden, _p(act), act_stride,
                                                  tokens, top_k, limit, _p(weights), _p(out_bf16), _p(out_f32), _p(ready),
                                                  _p(status), spins, _stream(stream)))


def launch_moe_slot_chain_fp4(x, x_stride, ids, views, inter, hidden, act, act_stride, tokens, top_k, limit, weights,
                              out_bf16, out_f32, ready, status, spins=0, stream=None, fp4_group=16):
    """Extension: the routed chain of a small decode batch in one launch (NVFP4 / MXFP4 experts)."""
    _check(_lib.load().dgpp_launch_moe_slot_chain_fp4(_p(x), x_stride, _p(ids), _p(views), inter, hidden, _p(act), act_stride,
                                                      tokens, top_k, limit, _p(weights), _p(out_bf16), _p(out_f32),
                                                      _p(ready), _p(status), spins, _stream(stream), fp4_group))


def launch_moe_select_slot_chain(scores, biased, ids, weights, cfg: MoeConfig, tokens, x, x_stride, views, inter, hidden, act,
                                 act_stride, limit, out_bf16, out_f32, ready, status, spins=0, stream=None):
    """Extension: selection + the routed chain in one launch for a one-token step (FP8; ids and weights are outputs)."""
    _check(_lib.load().dgpp_launch_moe_select_slot_chain(_p(scores), _p(biased), _p(ids), _p(weights), C.addressof(cfg), tokens,
                                                         _p(x), x_stride, _p(views), inter, hidden, _p(act), act_stride, limit,
                                                         _p(out_bf16), _p(out_f32), _p(ready), _p(status), spins,
                                                         _stream(stream)))


def launch_moe_select_slot_chain_fp4(scores, biased, ids, weights, cfg: MoeConfig, tokens, x, x_stride, views, inter, hidden,
                                     act, act_stride, limit, out_bf16, out_f32, ready, status, spins=0, stream=None,
                                     fp4_group=16):
    """Extension: selection + the routed chain in one launch for a one-token step (NVFP4 / MXFP4)."""
    _check(_lib.load().dgpp_launch_moe_select_slot_chain_fp4(_p(scores), _p(biased), _p(ids), _p(weights), C.addressof(cfg),
                                                             tokens, _p(x), x_stride, _p(views), inter, hidden, _p(act),
                                                             act_stride, limit, _p(out_bf16), _p(out_f32), _p(ready),
                                                             _p(status), spins, _stream(stream), fp4_group))


# ---- grouped twins ---------------------------------------------------------------------------------------
def launch_moe_grouped_gemv_bf16(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out,
                                 out_stride, n, k, stream=None):
    _check(_lib.load().dgpp_launch_moe_grouped_gemv_bf16(_p(act), act_stride, _p(segs), n_segs, max_rows,
                                                         rows_per_block, _p(views), which, _p(out), out_stride, n, k,
                                                         _stream(stream)))


def launch_moe_grouped_gemv_f32(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out,
                                out_stride, n, k, stream=None):
    _check(_lib.load().dgpp_launch_moe_grouped_gemv_f32(_p(act), act_stride, _p(segs), n_segs, max_rows,
                                                        rows_per_block, _p(views), which, _p(out), out_stride, n, k,
                                                        _stream(stream)))


def launch_moe_grouped_gemv_fp4_bf16(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out,
                                     out_stride, n, k, stream=None, fp4_group=16):
    _check(_lib.load().dgpp_launch_moe_grouped_gemv_fp4_bf16(_p(act), act_stride, _p(segs), n_segs, max_rows,
                                                             rows_per_block, _p(views), which, _p(out), out_stride, n,
                                                             k, _stream(stream), fp4_group))


def launch_moe_grouped_gemv_fp4_f32(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out,
                                    out_stride, n, k, stream=None, fp4_group=16):
    _check(_lib.load().dgpp_launch_moe_grouped_gemv_fp4_f32(_p(act), act_stride, _p(segs), n_segs, max_rows,
                                                            rows_per_block, _p(views), which, _p(out), out_stride, n,
                                                            k, _stream(stream), fp4_group))


# ---- dense projections --------------------------------------------------------------------------------------
def launch_fp4_gemv_bf16(act, act_row_stride_elems, w: Fp4Matrix, out, m, n, k, stream=None):
    _check(_lib.load().dgpp_launch_fp4_gemv_bf16(_p(act), act_row_stride_elems, C.addressof(w), _p(out), m, n, k,
                                                 _stream(stream)))


def launch_fp4_gemv_f32(act, act_row_stride_elems, w: Fp4Matrix, out, m, n, k, stream=None):
    _check(_lib.load().dgpp_launch_fp4_gemv_f32(_p(act), act_row_stride_elems, C.addressof(w), _p(out), m, n, k,
                                                _stream(stream)))


def fp4_gemv_accepts(w: Fp4Matrix) -> bool:
    return bool(_lib.load().dgpp_fp4_gemv_accepts(C.addressof(w)))


def launch_scale_gemm_bf16(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream=None,
                           out_row_stride_elems=0, mma_from_rows=0, ws=None, ws_bytes=0):
    _check(_lib.load().dgpp_launch_scale_gemm_bf16(_p(act), act_row_stride_elems, _p(w_payload), _p(w_scales), _p(out),
                                                   m, n, k, _stream(stream), out_row_stride_elems, mma_from_rows,
                                                   _p(ws), ws_bytes))


def launch_scale_gemm_f32(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream=None,
                          out_row_stride_elems=0, mma_from_rows=0, last_row_only=False, ws=None, ws_bytes=0,
                          compact_row=-1):
    _check(_lib.load().dgpp_launch_scale_gemm_f32(_p(act), act_row_stride_elems, _p(w_payload), _p(w_scales), _p(out),
                                                  m, n, k, _stream(stream), out_row_stride_elems, mma_from_rows,
                                                  1 if last_row_only else 0, _p(ws), ws_bytes, compact_row))


def launch_scale_gemm_grid_bf16(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream,
                                out_row_stride_elems, rs, cs, decode_mma=False, ws=None, ws_bytes=0,
                                prefill_tile=False):
    _check(_lib.load().dgpp_launch_scale_gemm_grid_bf16(_p(act), act_row_stride_elems, _p(w_payload), _p(w_scales),
                                                        _p(out), m, n, k, _stream(stream), out_row_stride_elems, rs,
                                                        cs, int(decode_mma), _p(ws), ws_bytes, int(prefill_tile)))


def launch_scale_gemm_grid_f32(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream,
                               out_row_stride_elems, rs, cs, decode_mma=False, ws=None, ws_bytes=0,
                               prefill_tile=False):
    _check(_lib.load().dgpp_launch_scale_gemm_grid_f32(_p(act), act_row_stride_elems, _p(w_payload), _p(w_scales),
                                                       _p(out), m, n, k, _stream(stream), out_row_stride_elems, rs,
                                                       cs, int(decode_mma), _p(ws), ws_bytes, int(prefill_tile)))


def launch_scale_gemm_grid_e8m0_bf16(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream,
                                     out_row_stride_elems, rs, cs, ws=None, ws_bytes=0, prefill_tile=False):
    _check(_lib.load().dgpp_launch_scale_gemm_grid_e8m0_bf16(_p(act), act_row_stride_elems, _p(w_payload),
                                                             _p(w_scales), _p(out), m, n, k, _stream(stream),
                                                             out_row_stride_elems, rs, cs, _p(ws), ws_bytes,
                                                             int(prefill_tile)))


def launch_scale_gemm_grid_e8m0_f32(act, act_row_stride_elems, w_payload, w_scales, out, m, n, k, stream,
                                    out_row_stride_elems, rs, cs, ws=None, ws_bytes=0, prefill_tile=False):
    _check(_lib.load().dgpp_launch_scale_gemm_grid_e8m0_f32(_p(act), act_row_stride_elems, _p(w_payload),
                                                            _p(w_scales), _p(out), m, n, k, _stream(stream),
                                                            out_row_stride_elems, rs, cs, _p(ws), ws_bytes,
                                                            int(prefill_tile)))


def launch_scale_gemv_multi_bf16(problems, act, act_row_stride_elems, rows, k, stream=None):
    arr = (Fp8GemvProblem * len(problems))(*problems)
    _check(_lib.load().dgpp_launch_scale_gemv_multi_bf16(C.addressof(arr), len(problems), _p(act),
                                                         act_row_stride_elems, rows, k, _stream(stream)))


def fp8_gemv_can_stage(w_payload, k) -> bool:
    return bool(_lib.load().dgpp_fp8_gemv_can_stage(_p(w_payload), k))


def launch_fp8_dequant_blocks(payload, scales, out_bf16, rows, cols, stream=None, rs=7, cs=7):
    _check(_lib.load().dgpp_launch_fp8_dequant_blocks(_p(payload), _p(scales), _p(out_bf16), rows, cols,
                                                      _stream(stream), rs, cs))


def launch_fp8_dequant_blocks_e8m0(payload, scales, out_bf16, rows, cols, stream, rs, cs):
    _check(_lib.load().dgpp_launch_fp8_dequant_blocks_e8m0(_p(payload), _p(scales), _p(out_bf16), rows, cols,
                                                           _stream(stream), rs, cs))


# ---- matrix-core launchers (src/kernels/glm_moe_launch.hpp:103-125, :311-345; src/kernels/mma_gemv.hpp:65-85) ----
def launch_dense_mma_bf16(act, act_stride, payload, scales, out, m, n, k, stream=None, out_stride=0):
    _check(_lib.load().dgpp_launch_dense_mma_bf16(_p(act), act_stride, _p(payload), _p(scales), _p(out), m, n, k,
                                                  _stream(stream), out_stride))


def launch_dense_mma_f32(act, act_stride, payload, scales, out, m, n, k, stream=None, out_stride=0):
    _check(_lib.load().dgpp_launch_dense_mma_f32(_p(act), act_stride, _p(payload), _p(scales), _p(out), m, n, k,
                                                 _stream(stream), out_stride))


def launch_dense_mma_fp4_bf16(act, act_stride, w: Fp4Matrix, out, m, n, k, stream=None):
    _check(_lib.load().dgpp_launch_dense_mma_fp4_bf16(_p(act), act_stride, C.addressof(w), _p(out), m, n, k, _stream(stream)))


def launch_dense_mma_fp4_f32(act, act_stride, w: Fp4Matrix, out, m, n, k, stream=None):
    _check(_lib.load().dgpp_launch_dense_mma_fp4_f32(_p(act), act_stride, C.addressof(w), _p(out), m, n, k, _stream(stream)))


def _mma_gemv(name, act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream, ws, ws_bytes):
    _check(getattr(_lib.load(), name)(_p(act), act_stride, _p(w), _p(scales), _p(out), m, n, k, out_stride, rs, cs,
                                      _stream(stream), _p(ws), ws_bytes))


def launch_mma_gemv_fp8_bf16(act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream=None, ws=None, ws_bytes=0):
    _mma_gemv("dgpp_launch_mma_gemv_fp8_bf16", act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream, ws, ws_bytes)


def launch_mma_gemv_fp8_f32(act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream=None, ws=None, ws_bytes=0):
    _mma_gemv("dgpp_launch_mma_gemv_fp8_f32", act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream, ws, ws_bytes)


def launch_mma_gemv_fp8e8m0_bf16(act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream=None, ws=None,
                                 ws_bytes=0):
    _mma_gemv("dgpp_launch_mma_gemv_fp8e8m0_bf16", act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream, ws,
              ws_bytes)


def launch_mma_gemv_fp8e8m0_f32(act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream=None, ws=None,
                                ws_bytes=0):
    _mma_gemv("dgpp_launch_mma_gemv_fp8e8m0_f32", act, act_stride, w, scales, out, m, n, k, out_stride, rs, cs, stream, ws,
              ws_bytes)


def launch_moe_grouped_mma_bf16(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, out_stride, n,
                                k, stream=None, act_rows=None):
    _check(_lib.load().dgpp_launch_moe_grouped_mma_bf16(_p(act), act_stride, _p(segs), n_segs, max_rows, rows_per_block,
                                                        _p(views), which, _p(out), out_stride, n, k, _stream(stream),
                                                        _p(act_rows)))


def launch_moe_grouped_mma_f32(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, out_stride, n, k,
                               stream=None, act_rows=None):
    _check(_lib.load().dgpp_launch_moe_grouped_mma_f32(_p(act), act_stride, _p(segs), n_segs, max_rows, rows_per_block,
                                                       _p(views), which, _p(out), out_stride, n, k, _stream(stream),
                                                       _p(act_rows)))


def mma_gemv_shape_ok(w, act, act_stride, m, k) -> bool:
    return bool(_lib.load().dgpp_mma_gemv_shape_ok(_p(w), _p(act), act_stride, m, k))


def mma_gemv_pair_ok(w0, w1, a0, a1, act_stride, m, n0, n1, k, ws, ws_bytes) -> bool:
    return bool(_lib.load().dgpp_mma_gemv_pair_ok(_p(w0), _p(w1), _p(a0), _p(a1), act_stride, m, n0, n1, k, _p(ws), ws_bytes))


def launch_mma_gemv_fp8_bf16_pair(a0, w0, s0, o0, n0, stride0, a1, w1, s1, o1, n1, stride1, act_stride, m, k, rs=7, cs=7,
                                  stream=None, ws=None, ws_bytes=0):
    _check(_lib.load().dgpp_launch_mma_gemv_fp8_bf16_pair(_p(a0), _p(w0), _p(s0), _p(o0), n0, stride0, _p(a1), _p(w1), _p(s1),
                                                          _p(o1), n1, stride1, act_stride, m, k, rs, cs, _stream(stream), _p(ws),
                                                          ws_bytes))


def launch_mma_gemv_fp8_swiglu_f32(gate, up, limit, act_stride, w, scales, out, m, n, k, out_stride=0, rs=7, cs=7,
                                   stream=None):
    _check(_lib.load().dgpp_launch_mma_gemv_fp8_swiglu_f32(_p(gate), _p(up), limit, act_stride, _p(w), _p(scales), _p(out),
                                                           m, n, k, out_stride, rs, cs, _stream(stream)))


def qwen_moe_shared_gate_bf16(x, g, w, tokens, hidden, stream=None):
    _check(_lib.load().dgpp_qwen_moe_shared_gate_bf16(_p(x), _p(g), _p(w), tokens, hidden, _stream(stream)))


def qwen_moe_shared_gate_up_decode_fp8(x, x_stride, gate_p, gate_s, up_p, up_s, g, act, sw, tokens, H, S, stream=None, rs=7,
                                       cs=7):
    _check(_lib.load().dgpp_qwen_moe_shared_gate_up_decode_fp8(_p(x), x_stride, _p(gate_p), _p(gate_s), _p(up_p), _p(up_s),
                                                               _p(g), _p(act), _p(sw), tokens, H, S, _stream(stream), rs, cs))


def qwen_moe_shared_down_decode_fp8(act, down_p, down_s, sw, acc, out, tokens, H, S, stream=None, rs=7, cs=7):
    _check(_lib.load().dgpp_qwen_moe_shared_down_decode_fp8(_p(act), _p(down_p), _p(down_s), _p(sw), _p(acc), _p(out), tokens,
                                                            H, S, _stream(stream), rs, cs))


def qwen_moe_shared_down_decode_routed_fp8(act, down_p, down_s, sw, contrib, weights, top_k, out, tokens, H, S, stream=None,
                                           rs=7, cs=7):
    _check(_lib.load().dgpp_qwen_moe_shared_down_decode_routed_fp8(_p(act), _p(down_p), _p(down_s), _p(sw), _p(contrib),
                                                                   _p(weights), top_k, _p(out), tokens, H, S,
                                                                   _stream(stream), rs, cs))


def qwen_moe_shared_tail_decode_fp8(x, x_stride, gate_p, gate_s, up_p, up_s, down_p, down_s, g, act, sw, acc, out, tokens, H, S,
                                    stream=None, rs=7, cs=7):
    _check(_lib.load().dgpp_qwen_moe_shared_tail_decode_fp8(_p(x), x_stride, _p(gate_p), _p(gate_s), _p(up_p), _p(up_s),
                                                            _p(down_p), _p(down_s), _p(g), _p(act), _p(sw), _p(acc), _p(out),
                                                            tokens, H, S, _stream(stream), rs, cs))


def qwen_moe_shared_tail_decode_routed_fp8(x, x_stride, gate_p, gate_s, up_p, up_s, down_p, down_s, g, act, sw, contrib, weights,
                                           top_k, out, tokens, H, S, stream=None, rs=7, cs=7):
    _check(_lib.load().dgpp_qwen_moe_shared_tail_decode_routed_fp8(_p(x), x_stride, _p(gate_p), _p(gate_s), _p(up_p), _p(up_s),
                                                                   _p(down_p), _p(down_s), _p(g), _p(act), _p(sw), _p(contrib),
                                                                   _p(weights), top_k, _p(out), tokens, H, S,
                                                                   _stream(stream), rs, cs))


def launch_mxfp8_quantize_rows(x, x_stride, rows, k, codes, scales, stream=None):
    _check(_lib.load().dgpp_launch_mxfp8_quantize_rows(_p(x), x_stride, rows, k, _p(codes), _p(scales), _stream(stream)))


def launch_minimax_swiglu_mxfp8_rows(gate, up, stride, rows, k, alpha, limit, codes, scales, stream=None):
    _check(_lib.load().dgpp_launch_minimax_swiglu_mxfp8_rows(_p(gate), _p(up), stride, rows, k, alpha, limit, _p(codes),
                                                             _p(scales), _stream(stream)))


def launch_mxfp8_gemm_bf16(a, a_scales, w, w_scales, out, m, n, k, stream=None, out_stride=0, output_tile=0):
    _check(_lib.load().dgpp_launch_mxfp8_gemm_bf16(_p(a), _p(a_scales), _p(w), _p(w_scales), _p(out), m, n, k,
                                                   _stream(stream), out_stride, output_tile))


def launch_mxfp8_gemm_f32(a, a_scales, w, w_scales, out, m, n, k, stream=None, out_stride=0, output_tile=0):
    _check(_lib.load().dgpp_launch_mxfp8_gemm_f32(_p(a), _p(a_scales), _p(w), _p(w_scales), _p(out), m, n, k,
                                                  _stream(stream), out_stride, output_tile))


def launch_dense_mma_fp4_prod_bf16(act, act_stride, seg, views, which, out, m, n, k, stream=None, fp4_group=16):
    _check(_lib.load().dgpp_launch_dense_mma_fp4_prod_bf16(_p(act), act_stride, _p(seg), _p(views), which, _p(out), m, n, k,
                                                           _stream(stream), fp4_group))


def launch_dense_mma_fp4_gate_up_bf16(act, act_stride, seg, views, gate, up, m, n, k, stream=None, fp4_group=16):
    _check(_lib.load().dgpp_launch_dense_mma_fp4_gate_up_bf16(_p(act), act_stride, _p(seg), _p(views), _p(gate), _p(up), m, n,
                                                              k, _stream(stream), fp4_group))


def launch_moe_grouped_mma_gate_up_swiglu(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, out, out_stride,
                                          n, k, limit, stream=None, act_rows=None):
    """Extension: grouped FP8 gate + up + SwiGLU in one matrix-core launch."""
    _check(_lib.load().dgpp_launch_moe_grouped_mma_gate_up_swiglu(_p(act), act_stride, _p(segs), n_segs, max_rows,
                                                                  rows_per_block, _p(views), _p(out), out_stride, n, k,
                                                                  limit, _stream(stream), _p(act_rows)))


def launch_moe_grouped_mma_gate_up_swiglu_fp4(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, out,
                                              out_stride, n, k, limit, stream=None, act_rows=None, fp4_group=16):
    """Extension: grouped NVFP4 / MXFP4 gate + up + SwiGLU in one matrix-core launch."""
    _check(_lib.load().dgpp_launch_moe_grouped_mma_gate_up_swiglu_fp4(_p(act), act_stride, _p(segs), n_segs, max_rows,
                                                                      rows_per_block, _p(views), _p(out), out_stride, n,
                                                                      k, limit, _stream(stream), _p(act_rows), fp4_group))


def launch_moe_grouped_mma_fp4_bf16(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, out_stride,
                                    n, k, stream=None, act_rows=None, fp4_group=16, tile_rows=64):
    _check(_lib.load().dgpp_launch_moe_grouped_mma_fp4_bf16(_p(act), act_stride, _p(segs), n_segs, max_rows, rows_per_block,
                                                            _p(views), which, _p(out), out_stride, n, k, _stream(stream),
                                                            _p(act_rows), fp4_group, tile_rows))


def launch_moe_grouped_mma_fp4_f32(act, act_stride, segs, n_segs, max_rows, rows_per_block, views, which, out, out_stride,
                                   n, k, stream=None, act_rows=None, fp4_group=16, tile_rows=64):
    _check(_lib.load().dgpp_launch_moe_grouped_mma_fp4_f32(_p(act), act_stride, _p(segs), n_segs, max_rows, rows_per_block,
                                                           _p(views), which, _p(out), out_stride, n, k, _stream(stream),
                                                           _p(act_rows), fp4_group, tile_rows))


def launch_mma_gemv_fp4_bf16(act, act_stride, w: Fp4Matrix, out, m, n, k, out_stride=0, stream=None, ws=None, ws_bytes=0):
    """Extension: the FP4 dense matrix-core form with an output stride and a split-K workspace."""
    _check(_lib.load().dgpp_launch_mma_gemv_fp4_bf16(_p(act), act_stride, C.addressof(w), _p(out), m, n, k, out_stride,
                                                     _stream(stream), _p(ws), ws_bytes))


def launch_mma_gemv_fp4_bf16_static(act, act_stride, w: Fp4Matrix, out, m, n, k, out_stride=0, stream=None):
    """Extension: launch_mma_gemv_fp4_bf16 on the library's own static workspace (allocates nothing)."""
    _check(_lib.load().dgpp_launch_mma_gemv_fp4_bf16_static(_p(act), act_stride, C.addressof(w), _p(out), m, n, k,
                                                            out_stride, _stream(stream)))


def static_scratch_release():
    """Frees the static workspace's binding to a stream (call once that stream's work is done)."""
    _check(_lib.load().dgpp_static_scratch_release())


def launch_mma_gemv_fp4_f32(act, act_stride, w: Fp4Matrix, out, m, n, k, out_stride=0, stream=None, ws=None, ws_bytes=0):
    _check(_lib.load().dgpp_launch_mma_gemv_fp4_f32(_p(act), act_stride, C.addressof(w), _p(out), m, n, k, out_stride,
                                                    _stream(stream), _p(ws), ws_bytes))


# ---- activation-quantized NVFP4 (W4A4) form: src/kernels/moe_w4a4.hpp ------------------------------------------------
def nvfp4_act_scale_stride(k: int) -> int:
    return _lib.load().dgpp_nvfp4_act_scale_stride(k)


def launch_quantize_rows_nvfp4(x, x_stride, rows, k, codes, scales, gs, stream=None, static_gs=0.0, static_gs_dev=None):
    _check(_lib.load().dgpp_launch_quantize_rows_nvfp4(_p(x), x_stride, rows, k, _p(codes), _p(scales), _p(gs), _stream(stream),
                                                       static_gs, _p(static_gs_dev)))


def launch_swiglu_quantize_rows_nvfp4(gate, up, stride, rows, k, limit, codes, scales, gs, stream=None, static_gs=0.0,
                                      static_gs_dev=None, qwen_rounding=False):
    _check(_lib.load().dgpp_launch_swiglu_quantize_rows_nvfp4(_p(gate), _p(up), stride, rows, k, limit, _p(codes), _p(scales),
                                                              _p(gs), _stream(stream), static_gs, _p(static_gs_dev),
                                                              1 if qwen_rounding else 0))


def launch_moe_grouped_w4a4_bf16(codes, scales, gs, act_rows, segs, n_segs, max_rows, views, which, out, out_stride, n, k,
                                 stream=None):
    _check(_lib.load().dgpp_launch_moe_grouped_w4a4_bf16(_p(codes), _p(scales), _p(gs), _p(act_rows), _p(segs), n_segs, max_rows,
                                                         _p(views), which, _p(out), out_stride, n, k, _stream(stream)))


def dense_w4a4_supported(k: int) -> bool:
    return bool(_lib.load().dgpp_dense_w4a4_supported(k))


def launch_dense_w4a4_bf16(a_codes, a_scales, a_scale_stride, a_gs, w_codes, w_scales, w_global, out, out_stride, m, n, k,
                           stream=None):
    _check(_lib.load().dgpp_launch_dense_w4a4_bf16(_p(a_codes), _p(a_scales), a_scale_stride, _p(a_gs), _p(w_codes), _p(w_scales),
                                                   _p(w_global), _p(out), out_stride, m, n, k, _stream(stream)))


def minimax_quantize_rows_nvfp4(x, stride, rows, k, codes, scales, globals_, stream=None):
    _check(_lib.load().dgpp_minimax_quantize_rows_nvfp4(_p(x), stride, rows, k, _p(codes), _p(scales), _p(globals_), _stream(stream)))


def minimax_swiglu_f32(gate, up, out, count, alpha, limit, stream=None):
    _check(_lib.load().dgpp_minimax_swiglu_f32(_p(gate), _p(up), _p(out), count, alpha, limit, _stream(stream)))


def launch_moe_accum_ordered_bf16down(out, down, down_stride, slot_row, slot_ids, slot_w, tokens, top_k, hidden, stream=None):
    _check(_lib.load().dgpp_launch_moe_accum_ordered_bf16down(_p(out), _p(down), down_stride, _p(slot_row), _p(slot_ids),
                                                              _p(slot_w), tokens, top_k, hidden, _stream(stream)))


def launch_moe_accum_ordered_f32_bf16down(out, down, down_stride, slot_row, slot_ids, slot_w, tokens, top_k, hidden, stream=None):
    _check(_lib.load().dgpp_launch_moe_accum_ordered_f32_bf16down(_p(out), _p(down), down_stride, _p(slot_row), _p(slot_ids),
                                                                  _p(slot_w), tokens, top_k, hidden, _stream(stream)))


def launch_moe_grouped_w4a4_f32(codes, scales, gs, act_rows, segs, n_segs, max_rows, views, which, out, out_stride, n, k,
                                stream=None):
    _check(_lib.load().dgpp_launch_moe_grouped_w4a4_f32(_p(codes), _p(scales), _p(gs), _p(act_rows), _p(segs), n_segs, max_rows,
                                                        _p(views), which, _p(out), out_stride, n, k, _stream(stream)))
