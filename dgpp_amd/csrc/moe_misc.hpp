// Host entry points of the router (moe_router.hip), grouping (moe_grouping.hip) and elementwise / accumulation
// (moe_elementwise.hip) kernels. Arguments are
// validated by the C ABI layer; these only pick grids and launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/dgpp_amd.h"

namespace dgpp_amd {

hipError_t run_hash_routes(const int64_t* tokens, const int32_t* tid2eid, const float* scores, int32_t* ids, float* weights,
                           int n_tokens, int vocab, int n_experts, int top_k, float scaling, int norm_topk, hipStream_t stream);
hipError_t run_router_dots(int mode, const uint16_t* hidden, const uint16_t* gate, const float* bias, float* scores,
                           float* biased, int tokens, int hidden_dim, int n_experts, hipStream_t stream, int allow_tiled = 1);
hipError_t run_router_select(int mode, const float* scores, const float* biased, int32_t* ids, float* weights,
                             int tokens, int n_experts, int top_k, float scaling, int norm_topk, hipStream_t stream);
hipError_t run_minimax_router(const uint16_t* x, const float* gate, const float* bias, int rows, int hidden, int experts,
                              int top_k, float factor, float* scores, int32_t* ids, float* weights, hipStream_t stream);
// tokens <= 16, n_experts <= 512, top_k <= 16; order may be null (selection only).
hipError_t run_router_select_order(int mode, const float* scores, const float* biased, int32_t* ids, float* weights,
                                   int32_t* order, int tokens, int n_experts, int top_k, float scaling, int norm_topk,
                                   int shared_early, hipStream_t stream);
hipError_t run_swiglu_clamp(const uint16_t* gate, const uint16_t* up, uint16_t* out, int64_t n, float limit,
                            hipStream_t stream);
hipError_t run_gather_rows(const uint16_t* src, const int32_t* rows, uint16_t* dst, int n_rows, int hidden,
                           hipStream_t stream);
hipError_t run_accum(float* acc, const float* y, const int32_t* rows, const float* row_w, int n_rows, int hidden,
                     hipStream_t stream);
hipError_t run_round_bf16(uint16_t* out, const float* acc, int64_t n, hipStream_t stream);
hipError_t run_slot_accum(void* out, int out_f32, int with_shared, const float* contrib, const float* weights,
                          int tokens, int hidden, int top_k, hipStream_t stream);
// down_bf16 != 0: the rows at `down` are BF16 (down_stride in BF16 elements).
hipError_t run_accum_ordered(void* out, int out_f32, const void* down, int down_bf16, size_t down_stride,
                             const int32_t* slot_row, const int32_t* slot_ids, const float* slot_w, int shared_row0, int tokens,
                             int top_k, int hidden, hipStream_t stream);
hipError_t run_segment(const int32_t* ids, int tokens, int top_k, int n_experts, int32_t* rows, int32_t* slot_row,
                       DgppMoeSegment* segs, hipStream_t stream);
hipError_t run_slot_order(const int32_t* ids, int32_t* order, int32_t* runs, int slots, int top_k, int n_experts,
                          int shared_early, hipStream_t stream);
hipError_t run_tile_list(const DgppMoeSegment* segs, int n_segs, int tile_rows, DgppMoeTile* tiles, int32_t* count,
                         hipStream_t stream);
hipError_t run_compact_segments(const DgppMoeSegment* input, DgppMoeSegment* output, int experts, int capacity,
                                hipStream_t stream);
hipError_t run_probe_copy(void* dst, const void* src, size_t bytes, hipStream_t stream);
// sink: at least 8192 words, never written in practice (keeps the loads alive)
hipError_t run_probe_read(const void* src, size_t bytes, void* sink, int nontemporal, int blocks, int span, hipStream_t stream);
hipError_t run_fp8_dequant(const uint8_t* payload, const void* scales, int e8m0, uint16_t* out, int64_t rows,
                           int64_t cols, int rs, int cs, hipStream_t stream);

}  // namespace dgpp_amd
