"""ctypes binding of libdgpp_amd.so: the C ABI declared in include/dgpp_amd.h.

Loading fails loudly when the library has not been built; nothing here falls back to a CPU path.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

PKG = Path(__file__).resolve().parent
LIB_PATH = PKG / "lib" / "libdgpp_amd.so"

OK, INVALID_ARGUMENT, RUNTIME_ERROR = 0, 1, 2


class MoeExpertView(C.Structure):
    """Device expert-table entry; 96 bytes, the reference's MoeExpertView layout
    (src/models/glm/moe.hpp:232-292)."""
    _fields_ = [
        ("payload", C.c_void_p), ("scales", C.c_void_p), ("fp4_scales", C.c_void_p),
        ("fp4_global", C.c_void_p), ("scale_shift_rows", C.c_int32), ("scale_shift_cols", C.c_int32),
        ("fp4_group", C.c_int32), ("reserved0", C.c_int32), ("reserved1", C.c_void_p),
        ("reserved2", C.c_int32 * 2), ("reserved3", C.c_void_p * 2), ("reserved4", C.c_int32 * 4),
    ]


class MoeSegment(C.Structure):
    _fields_ = [("row0", C.c_int32), ("rows", C.c_int32), ("expert", C.c_int32)]


class MoeTile(C.Structure):
    _fields_ = [("seg", C.c_int32), ("m0", C.c_int32)]


class Fp4Matrix(C.Structure):
    """src/models/quant_matrix.hpp:117-138 (GlmFp4Matrix)."""
    _fields_ = [
        ("payload", C.c_void_p), ("scales", C.c_void_p), ("global_scale", C.c_void_p),
        ("rows", C.c_int64), ("cols", C.c_int64), ("scale_group", C.c_int32), ("reserved0", C.c_int32),
        ("reserved1", C.c_void_p),
    ]


class MoeConfig(C.Structure):
    """The router-relevant fields of GlmMoeConfig (src/models/glm/moe.hpp:51-134)."""
    _fields_ = [
        ("hidden", C.c_int32), ("inter", C.c_int32), ("n_experts", C.c_int32), ("top_k", C.c_int32),
        ("n_shared_experts", C.c_int32), ("routed_scaling_factor", C.c_float), ("norm_topk_prob", C.c_int32),
        ("swiglu_limit", C.c_float), ("router_mode", C.c_int32),
    ]


class Fp8GemvProblem(C.Structure):
    _fields_ = [
        ("payload", C.c_void_p), ("scales", C.c_void_p), ("out", C.c_void_p), ("n", C.c_int32),
        ("reserved0", C.c_int32), ("out_stride", C.c_size_t), ("rs", C.c_int32), ("cs", C.c_int32),
        ("bf16_weight", C.c_void_p),
    ]


assert C.sizeof(MoeExpertView) == 96 and C.sizeof(MoeSegment) == 12 and C.sizeof(Fp4Matrix) == 56

_P, _I, _F, _Z, _L = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_int64

# name -> (restype, argtypes). Every `dgpp_*` function of include/dgpp_amd.h appears here.
SIGNATURES = {
    "dgpp_last_error": (C.c_char_p, []),
    "dgpp_target_arch": (C.c_char_p, []),
    "dgpp_moe_config_validate": (_I, [_P]),
    "dgpp_launch_moe_router": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _I]),
    "dgpp_launch_moe_router_select": (_I, [_P, _P, _P, _P, _P, _I, _P]),
    "dgpp_launch_moe_router_select_order": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _P]),
    "dgpp_dense_fp4_decode_shape": (_I, [_I, _I, _I, _I]),
    "dgpp_try_dense_fp4_decode_bf16": (_I, [_P, _Z, _P, _P, _I, _P, _I, _I, _I, _P, _I, _P]),
    "dgpp_launch_scale_gemm_tile_bf16": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _P, _I, _I]),
    "dgpp_launch_scale_gemm_tile_f32": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _P, _I, _I]),
    "dgpp_launch_moe_slot_gate_up_swiglu_mixed": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _I, _I, _F, _I, _I,
                                                        _P, _I, _I]),
    "dgpp_mma_gemv_shape_ok": (_I, [_P, _P, _Z, _I, _I]),
    "dgpp_mma_gemv_pair_ok": (_I, [_P, _P, _P, _P, _Z, _I, _I, _I, _I, _P, _Z]),
    "dgpp_launch_mma_gemv_fp8_bf16_pair": (_I, [_P, _P, _P, _P, _I, _Z, _P, _P, _P, _P, _I, _Z, _Z, _I, _I, _I, _I, _P, _P, _Z]),
    "dgpp_launch_moe_hash_routes": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _P]),
    "dgpp_launch_moe_router_dots": (_I, [_P, _P, _P, _P, _P, _P, _I, _P]),
    "dgpp_launch_moe_select_gate_up_swiglu": (_I, [_P, _P, _P, _P, _P, _I, _P, _Z, _P, _I, _I, _P, _I, _F, _P]),
    "dgpp_launch_moe_select_gate_up_swiglu_fp4": (_I, [_P, _P, _P, _P, _P, _I, _P, _Z, _P, _I, _I, _P, _I, _F, _P, _I]),
    "dgpp_launch_moe_swiglu_clamp": (_I, [_P, _P, _P, _L, _F, _P]),
    "dgpp_launch_moe_gather_rows": (_I, [_P, _P, _P, _I, _I, _P]),
    "dgpp_launch_moe_accum": (_I, [_P, _P, _P, _P, _I, _I, _P]),
    "dgpp_launch_moe_round_bf16": (_I, [_P, _P, _L, _P]),
    "dgpp_launch_moe_segment": (_I, [_P, _I, _I, _I, _P, _P, _P, _P]),
    "dgpp_moe_tile_list_capacity": (_I, [_I, _I, _I]),
    "dgpp_launch_moe_tile_list": (_I, [_P, _I, _I, _P, _P, _P]),
    "dgpp_moe_run_groups_max": (_I, [_I]),
    "dgpp_launch_moe_slot_order": (_I, [_P, _P, _I, _I, _I, _P, _I, _P]),
    "dgpp_minimax_compact_segments": (_I, [_P, _P, _I, _I, _P]),
    "dgpp_minimax_router": (_I, [_P, _P, _P, _I, _I, _I, _I, _F, _P, _P, _P, _P]),
    "dgpp_launch_moe_accum_ordered": (_I, [_P, _P, _Z, _P, _P, _P, _I, _I, _I, _I, _P]),
    "dgpp_launch_moe_accum_ordered_f32": (_I, [_P, _P, _Z, _P, _P, _P, _I, _I, _I, _I, _P]),
    "dgpp_launch_moe_accum_ordered_bf16down": (_I, [_P, _P, _Z, _P, _P, _P, _I, _I, _I, _P]),
    "dgpp_launch_moe_accum_ordered_f32_bf16down": (_I, [_P, _P, _Z, _P, _P, _P, _I, _I, _I, _P]),
    "dgpp_launch_moe_slot_accum": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "dgpp_launch_moe_slot_accum_routed_f32": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "dgpp_launch_moe_slot_accum_routed_bf16": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "dgpp_launch_moe_slot_gate_up_swiglu": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _I, _I, _F, _P, _I, _I]),
    "dgpp_launch_moe_slot_down": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _I, _I, _I, _P, _I, _I]),
    "dgpp_launch_moe_slot_gate_up_swiglu_fp4": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _I, _I, _F, _P, _I, _I, _I, _I]),
    "dgpp_launch_moe_slot_down_fp4": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _I, _I, _I, _P, _I, _I, _I, _I, _P]),
    "dgpp_launch_moe_slot_gate_up_swiglu_ex": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _I, _I, _F, _P, _I, _I, _I]),
    "dgpp_launch_moe_slot_down_ex": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _I, _I, _I, _P, _I, _I, _I, _P, _P]),
    "dgpp_launch_moe_slot_gate_up_swiglu_fp4_ex": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _I, _I, _F, _P, _I, _I, _I, _I, _I]),
    "dgpp_launch_moe_slot_down_fp4_ex": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _I, _I, _I, _P, _I, _I, _I, _I, _P, _I, _P, _P]),
    "dgpp_launch_moe_slot_down_accum": (_I, [_P, _Z, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P]),
    "dgpp_launch_moe_slot_down_accum_fp4": (_I, [_P, _Z, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _I]),
    "dgpp_moe_slot_chain_ready_bytes": (C.c_size_t, [_I, _I]),
    "dgpp_launch_moe_slot_chain": (_I, [_P, _Z, _P, _P, _I, _I, _P, _I, _I, _I, _F, _P, _P, _P, _P, _P, C.c_uint, _P]),
    "dgpp_launch_moe_select_slot_chain": (_I, [_P, _P, _P, _P, _P, _I, _P, _Z, _P, _I, _I, _P, _I, _F, _P, _P, _P, _P, C.c_uint,
                                               _P]),
    "dgpp_launch_moe_select_slot_chain_fp4": (_I, [_P, _P, _P, _P, _P, _I, _P, _Z, _P, _I, _I, _P, _I, _F, _P, _P, _P, _P,
                                                   C.c_uint, _P, _I]),
    "dgpp_launch_moe_slot_chain_fp4": (_I, [_P, _Z, _P, _P, _I, _I, _P, _I, _I, _I, _F, _P, _P, _P, _P, _P, C.c_uint, _P,
                                            _I]),
    "dgpp_launch_dense_mma_bf16": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _P, _Z]),
    "dgpp_launch_dense_mma_f32": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _P, _Z]),
    "dgpp_launch_dense_mma_fp4_bf16": (_I, [_P, _Z, _P, _P, _I, _I, _I, _P]),
    "dgpp_launch_dense_mma_fp4_f32": (_I, [_P, _Z, _P, _P, _I, _I, _I, _P]),
    "dgpp_launch_mma_gemv_fp4_bf16": (_I, [_P, _Z, _P, _P, _I, _I, _I, _Z, _P, _P, _Z]),
    "dgpp_launch_mma_gemv_fp4_f32": (_I, [_P, _Z, _P, _P, _I, _I, _I, _Z, _P, _P, _Z]),
    "dgpp_launch_mma_gemv_fp4_bf16_static": (_I, [_P, _Z, _P, _P, _I, _I, _I, _Z, _P]),
    "dgpp_static_scratch_release": (_I, []),
    "dgpp_launch_mma_gemv_fp8_bf16": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _Z, _I, _I, _P, _P, _Z]),
    "dgpp_launch_mma_gemv_fp8_f32": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _Z, _I, _I, _P, _P, _Z]),
    "dgpp_launch_mma_gemv_fp8e8m0_bf16": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _Z, _I, _I, _P, _P, _Z]),
    "dgpp_launch_mma_gemv_fp8e8m0_f32": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _Z, _I, _I, _P, _P, _Z]),
    "dgpp_launch_moe_grouped_mma_bf16": (_I, [_P, _Z, _P, _I, _I, _I, _P, _I, _P, _Z, _I, _I, _P, _P]),
    "dgpp_launch_moe_grouped_mma_f32": (_I, [_P, _Z, _P, _I, _I, _I, _P, _I, _P, _Z, _I, _I, _P, _P]),
    "dgpp_launch_mma_gemv_fp8_swiglu_f32": (_I, [_P, _P, _F, _Z, _P, _P, _P, _I, _I, _I, _Z, _I, _I, _P]),
    "dgpp_qwen_moe_shared_gate_bf16": (_I, [_P, _P, _P, _I, _I, _P]),
    "dgpp_qwen_moe_shared_gate_up_decode_fp8": (_I, [_P, _Z, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P, _I, _I]),
    "dgpp_qwen_moe_shared_down_decode_fp8": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _P, _I, _I]),
    "dgpp_qwen_moe_shared_down_decode_routed_fp8": (_I, [_P, _P, _P, _P, _P, _P, _I, _P, _I, _I, _I, _P, _I, _I]),
    "dgpp_qwen_moe_shared_tail_decode_fp8": (_I, [_P, _Z, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P, _I, _I]),
    "dgpp_qwen_moe_shared_tail_decode_routed_fp8": (_I, [_P, _Z, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _I, _I,
                                                         _I, _P, _I, _I]),
    "dgpp_nvfp4_act_scale_stride": (C.c_size_t, [_I]),
    "dgpp_launch_quantize_rows_nvfp4": (_I, [_P, _Z, _I, _I, _P, _P, _P, _P, _F, _P]),
    "dgpp_launch_swiglu_quantize_rows_nvfp4": (_I, [_P, _P, _Z, _I, _I, _F, _P, _P, _P, _P, _F, _P, _I]),
    "dgpp_launch_moe_grouped_w4a4_bf16": (_I, [_P, _P, _P, _P, _P, _I, _I, _P, _I, _P, _Z, _I, _I, _P]),
    "dgpp_launch_moe_grouped_w4a4_f32": (_I, [_P, _P, _P, _P, _P, _I, _I, _P, _I, _P, _Z, _I, _I, _P]),
    "dgpp_dense_w4a4_supported": (_I, [_I]),
    "dgpp_launch_dense_w4a4_bf16": (_I, [_P, _P, _Z, _P, _P, _P, _P, _P, _Z, _I, _I, _I, _P]),
    "dgpp_minimax_quantize_rows_nvfp4": (_I, [_P, _Z, _I, _I, _P, _P, _P, _P]),
    "dgpp_minimax_swiglu_f32": (_I, [_P, _P, _P, C.c_int64, _F, _F, _P]),
    "dgpp_launch_mxfp8_quantize_rows": (_I, [_P, _Z, _I, _I, _P, _P, _P]),
    "dgpp_launch_minimax_swiglu_mxfp8_rows": (_I, [_P, _P, _Z, _I, _I, _F, _F, _P, _P, _P]),
    "dgpp_launch_mxfp8_gemm_bf16": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _P, _Z, _I]),
    "dgpp_launch_mxfp8_gemm_f32": (_I, [_P, _P, _P, _P, _P, _I, _I, _I, _P, _Z, _I]),
    "dgpp_launch_dense_mma_fp4_prod_bf16": (_I, [_P, _Z, _P, _P, _I, _P, _I, _I, _I, _P, _I]),
    "dgpp_launch_dense_mma_fp4_gate_up_bf16": (_I, [_P, _Z, _P, _P, _P, _P, _I, _I, _I, _P, _I]),
    "dgpp_launch_moe_grouped_mma_gate_up_swiglu": (_I, [_P, _Z, _P, _I, _I, _I, _P, _P, _Z, _I, _I, _F, _P, _P]),
    "dgpp_launch_moe_grouped_mma_gate_up_swiglu_fp4": (_I, [_P, _Z, _P, _I, _I, _I, _P, _P, _Z, _I, _I, _F, _P, _P, _I]),
    "dgpp_launch_moe_grouped_mma_fp4_bf16": (_I, [_P, _Z, _P, _I, _I, _I, _P, _I, _P, _Z, _I, _I, _P, _P, _I, _I]),
    "dgpp_launch_moe_grouped_mma_fp4_f32": (_I, [_P, _Z, _P, _I, _I, _I, _P, _I, _P, _Z, _I, _I, _P, _P, _I, _I]),
    "dgpp_launch_moe_grouped_gemv_bf16": (_I, [_P, _Z, _P, _I, _I, _I, _P, _I, _P, _Z, _I, _I, _P]),
    "dgpp_launch_moe_grouped_gemv_f32": (_I, [_P, _Z, _P, _I, _I, _I, _P, _I, _P, _Z, _I, _I, _P]),
    "dgpp_launch_moe_grouped_gemv_fp4_bf16": (_I, [_P, _Z, _P, _I, _I, _I, _P, _I, _P, _Z, _I, _I, _P, _I]),
    "dgpp_launch_moe_grouped_gemv_fp4_f32": (_I, [_P, _Z, _P, _I, _I, _I, _P, _I, _P, _Z, _I, _I, _P, _I]),
    "dgpp_launch_fp4_gemv_bf16": (_I, [_P, _Z, _P, _P, _I, _I, _I, _P]),
    "dgpp_launch_fp4_gemv_f32": (_I, [_P, _Z, _P, _P, _I, _I, _I, _P]),
    "dgpp_fp4_gemv_accepts": (_I, [_P]),
    "dgpp_launch_scale_gemm_bf16": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _P, _Z, _I, _P, _Z]),
    "dgpp_launch_scale_gemm_f32": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _P, _Z, _I, _I, _P, _Z, _I]),
    "dgpp_launch_scale_gemm_grid_bf16": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _P, _Z, _I, _I, _I, _P, _Z, _I]),
    "dgpp_launch_scale_gemm_grid_f32": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _P, _Z, _I, _I, _I, _P, _Z, _I]),
    "dgpp_launch_scale_gemm_grid_e8m0_bf16": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _P, _Z, _I, _I, _P, _Z, _I]),
    "dgpp_launch_scale_gemm_grid_e8m0_f32": (_I, [_P, _Z, _P, _P, _P, _I, _I, _I, _P, _Z, _I, _I, _P, _Z, _I]),
    "dgpp_launch_scale_gemv_multi_bf16": (_I, [_P, _I, _P, _Z, _I, _I, _P]),
    "dgpp_fp8_gemv_can_stage": (_I, [_P, _I]),
    "dgpp_launch_fp8_dequant_blocks": (_I, [_P, _P, _P, _L, _L, _P, _I, _I]),
    "dgpp_launch_fp8_dequant_blocks_e8m0": (_I, [_P, _P, _P, _L, _L, _P, _I, _I]),
    "dgpp_bf16_to_f32": (_F, [C.c_uint16]),
    "dgpp_f32_to_bf16": (C.c_uint16, [_F]),
    "dgpp_e4m3_to_f32": (_F, [C.c_uint8]),
    "dgpp_f32_to_e4m3": (C.c_uint8, [_F]),
    "dgpp_e2m1_to_f32": (_F, [C.c_uint8]),
    "dgpp_f32_to_e2m1": (C.c_uint8, [_F]),
    "dgpp_e8m0_to_f32": (_F, [C.c_uint8]),
    "dgpp_e8m0_ceil_log2": (C.c_uint8, [_F]),
    "dgpp_encode_fp8_blocks": (None, [_P, _L, _L, _I, _I, _P, _P, _I]),
    "dgpp_encode_nvfp4": (_F, [_P, _L, _L, _P, _P, _I]),
    "dgpp_encode_mxfp4": (None, [_P, _L, _L, _P, _P, _I]),
    "dgpp_encode_mxfp8": (None, [_P, _L, _L, _P, _P, _I]),
    "dgpp_fill_normal_f32": (None, [C.c_uint64, _F, _F, _L, _P, _I]),
    "dgpp_fill_normal_bf16": (None, [C.c_uint64, _F, _F, _L, _P, _I]),
    "dgpp_fill_zipf_routes": (None, [C.c_uint64, C.c_double, _I, _I, _I, _P]),
}



class MoeLayerDesc(C.Structure):
    """include/dgpp_amd_layer.h: DgppMoeLayerDesc."""
    _fields_ = [
        ("cfg", MoeConfig), ("expert_format", C.c_int32), ("max_tokens", C.c_int32), ("views", C.c_void_p),
        ("shared_in_table", C.c_int32), ("shared_inter", C.c_int32), ("sh_payload", C.c_void_p * 3),
        ("sh_scales", C.c_void_p * 3), ("sh_rs", C.c_int32), ("sh_cs", C.c_int32), ("router_gate", C.c_void_p),
        ("router_bias", C.c_void_p), ("sh_scales_e8m0", C.c_void_p * 3),
    ]


class MoeResidentDesc(C.Structure):
    """include/dgpp_amd_layer.h: DgppMoeResidentDesc."""
    _fields_ = [
        ("cfg", MoeConfig), ("max_tokens", C.c_int32), ("rank", C.c_int32), ("world", C.c_int32), ("routed", C.c_void_p),
        ("shared", C.c_void_p), ("shared_inter", C.c_int64), ("router_weight", C.c_void_p), ("router_bias", C.c_void_p),
    ]


# include/dgpp_amd_layer.h
LAYER_SIGNATURES = {
    "dgpp_moe_layer_last_error": (C.c_char_p, []),
    "dgpp_moe_layer_scratch_bytes": (C.c_size_t, [_P, _I, _I]),
    "dgpp_moe_layer_scratch_bytes_dense_shared": (C.c_size_t, [_P, _I, _I]),
    "dgpp_moe_layer_create": (_I, [_P, _P]),
    "dgpp_moe_layer_destroy": (None, [_P]),
    "dgpp_moe_layer_enqueue_decode": (_I, [_P, _P, _Z, _P, _P, _I, _P]),
    "dgpp_moe_layer_enqueue_decode_scores": (_I, [_P, _P, _Z, _P, _P, _P, _P, _I, _P]),
    "dgpp_moe_layer_enqueue_decode_routed": (_I, [_P, _P, _Z, _P, _P, _P, _P, _I, _P]),
    "dgpp_moe_layer_enqueue_grouped_routed": (_I, [_P, _P, _Z, _P, _P, _P, _P, _I, _P]),
    "dgpp_moe_layer_enqueue_prefill_routed": (_I, [_P, _P, _Z, _P, _P, _P, _P, _I, _P]),
    "dgpp_moe_layer_enqueue_prefill": (_I, [_P, _P, _Z, _P, _P, _I, _P]),
    "dgpp_moe_layer_route_prefill_rows": (_I, [_P, _P, _Z, _I, _I, _P]),
    "dgpp_moe_layer_enqueue_prefill_phased": (_I, [_P, _P, _Z, _I, _P]),
    "dgpp_moe_layer_accumulate_prefill_rows": (_I, [_P, _P, _P, _I, _I, _I, _P]),
    "dgpp_moe_layer_enqueue_prefill_routed_w4a4": (_I, [_P, _P, _Z, _P, _P, _P, _P, _I, _P, _P, _I]),
    "dgpp_moe_resident_last_error": (C.c_char_p, []),
    "dgpp_moe_resident_load": (_I, [_P, _P]),
    "dgpp_moe_resident_destroy": (None, [_P]),
    "dgpp_moe_resident_layer": (_P, [_P]),
    "dgpp_moe_resident_weight_bytes": (C.c_size_t, [_P]),
    "dgpp_moe_resident_inter": (_I, [_P]),
    "dgpp_moe_layer_views": (_P, [_P]),
    "dgpp_moe_layer_check": (_I, [_P, _P]),
    "dgpp_moe_layer_ids": (_P, [_P]),
    "dgpp_moe_layer_weights": (_P, [_P]),
}

# include/dgpp_amd_bench.h (measurement aids; not part of the launcher surface)
BENCH_SIGNATURES = {
    "dgpp_tune_set": (None, [_I, _I]),
    "dgpp_tune_get": (_I, [_I]),
    "dgpp_tune_enabled": (_I, []),
    "dgpp_probe_copy": (_I, [_P, _P, C.c_size_t, _P]),
    "dgpp_probe_read": (_I, [_P, C.c_size_t, _P, _I, _I, _I, _P]),
}

_lib = None


def load() -> C.CDLL:
    """Loads the built library (once) and types every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m dgpp_amd.build` "
            "(there is no CPU fallback for the HIP path)")
    # One HIP runtime per process: PyTorch ships its own copy, and a process that uses both (tests, the bench)
    # must let PyTorch load it first; this library then binds to the copy already in the process.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(str(LIB_PATH))
    for name, (res, args) in {**SIGNATURES, **LAYER_SIGNATURES, **BENCH_SIGNATURES}.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
